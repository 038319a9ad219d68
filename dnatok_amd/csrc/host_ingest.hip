// Host-side ingest helpers: what a caller does to its strings before the bytes cross PCIe.
// Plain CPU code (no device work): one pass over the bytes instead of one numpy pass per rule.
#include "common.hpp"

#include <string.h>

namespace dnatok {

struct IngestTables {
    uint8_t code[256];      // ASCII -> 2-bit code; everything but C G T (either case) is 0, like A
    uint8_t upper[256];     // a-z -> A-Z
    uint8_t valid_upper[256];
    uint8_t valid_both[256];
    IngestTables()
    {
        for (int i = 0; i < 256; ++i) {
            code[i] = 0;
            upper[i] = (uint8_t)((i >= 'a' && i <= 'z') ? i - 32 : i);
            valid_upper[i] = 0;
            valid_both[i] = 0;
        }
        const char *acgtn = "ACGTN";
        for (int j = 0; j < 5; ++j) {
            valid_upper[(int)acgtn[j]] = 1;
            valid_both[(int)acgtn[j]] = 1;
            valid_both[(int)acgtn[j] + 32] = 1;
        }
        code['C'] = code['c'] = 1;
        code['G'] = code['g'] = 2;
        code['T'] = code['t'] = 3;
    }
};

static const IngestTables &ingest_tables()
{
    static const IngestTables t;
    return t;
}

}  // namespace dnatok

using namespace dnatok;

extern "C" int dnatok_host_clean_ascii(uint8_t *bytes_h, int64_t n, int upper_case, int invalid_to_n,
                                       int64_t *n_replaced)
{
    DNATOK_REQUIRE(n >= 0, DNATOK_E_INVALID, "dnatok_host_clean_ascii: negative size");
    DNATOK_REQUIRE(bytes_h || n == 0, DNATOK_E_INVALID, "dnatok_host_clean_ascii: null buffer");
    const IngestTables &t = ingest_tables();
    const uint8_t *valid = upper_case ? t.valid_upper : t.valid_both;
    int64_t replaced = 0;
    for (int64_t i = 0; i < n; ++i) {
        uint8_t c = bytes_h[i];
        if (upper_case) c = t.upper[c];
        if (invalid_to_n && !valid[c]) {
            c = 'N';
            ++replaced;
        }
        bytes_h[i] = c;
    }
    if (n_replaced) *n_replaced = replaced;
    return DNATOK_OK;
}

extern "C" int dnatok_host_pack_2bit(const uint8_t *ascii_h, int64_t n_rows, int64_t row_len,
                                     uint8_t *packed_h)
{
    DNATOK_REQUIRE(n_rows >= 0 && row_len >= 0, DNATOK_E_INVALID, "dnatok_host_pack_2bit: negative size");
    if (n_rows == 0 || row_len == 0) return DNATOK_OK;
    DNATOK_REQUIRE(ascii_h && packed_h, DNATOK_E_INVALID, "dnatok_host_pack_2bit: null buffer");
    const uint8_t *code = ingest_tables().code;
    const int64_t row_packed = (row_len + 3) / 4;
    const int64_t whole = row_len / 4;
    for (int64_t b = 0; b < n_rows; ++b) {
        const uint8_t *src = ascii_h + b * row_len;
        uint8_t *dst = packed_h + b * row_packed;
        for (int64_t q = 0; q < whole; ++q) {
            const uint8_t *c = src + q * 4;
            dst[q] = (uint8_t)(code[c[0]] | (code[c[1]] << 2) | (code[c[2]] << 4) | (code[c[3]] << 6));
        }
        if (whole < row_packed) {                      // last, partial group: missing bases are code 0
            uint8_t v = 0;
            for (int64_t k = whole * 4; k < row_len; ++k) v |= (uint8_t)(code[src[k]] << (2 * (k - whole * 4)));
            dst[whole] = v;
        }
    }
    return DNATOK_OK;
}

// FASTA text -> the bytes of all records laid end to end + offsets, in one pass over the text.
// With seq_out == NULL only the counts are produced (the sizes the second call needs).
extern "C" int dnatok_host_fasta_scan(const uint8_t *text_h, int64_t n, int upper_case, uint8_t *seq_out,
                                      int64_t seq_capacity, int64_t *offsets_out, int64_t *name_spans_out,
                                      int64_t max_records, int64_t *n_records, int64_t *n_bases)
{
    DNATOK_REQUIRE(n >= 0 && (text_h || n == 0), DNATOK_E_INVALID, "dnatok_host_fasta_scan: bad text buffer");
    DNATOK_REQUIRE(n_records && n_bases, DNATOK_E_INVALID, "dnatok_host_fasta_scan: null count pointer");
    const bool writing = seq_out != nullptr;
    DNATOK_REQUIRE(!writing || offsets_out, DNATOK_E_INVALID, "dnatok_host_fasta_scan: offsets needed with seq_out");
    int64_t rec = 0, bases = 0;
    bool open_record = false;                          // a record has begun (by a header, or by bases without one)
    auto begin_record = [&](int64_t name_lo, int64_t name_hi) -> bool {
        if (writing) {
            if (rec >= max_records) return false;
            offsets_out[rec] = bases;
            if (name_spans_out) { name_spans_out[2 * rec] = name_lo; name_spans_out[2 * rec + 1] = name_hi; }
        }
        ++rec;
        open_record = true;
        return true;
    };
    // Line by line; the line feeds are found and whole lines are copied by the C library's
    // vectorised routines, and only a line that holds a blank, a tab or a stray carriage return
    // is copied byte by byte.
    int64_t i = 0;
    while (i < n) {
        const uint8_t *nl = static_cast<const uint8_t *>(memchr(text_h + i, '\n', (size_t)(n - i)));
        const int64_t e = nl ? nl - text_h : n;            // the line is [i, e)
        int64_t line_end = e;
        if (line_end > i && text_h[line_end - 1] == '\r') --line_end;
        const int64_t len = line_end - i;
        if (len > 0 && text_h[i] == '>') {
            DNATOK_REQUIRE(begin_record(i + 1, line_end), DNATOK_E_TOO_LARGE,
                           "dnatok_host_fasta_scan: more than %lld records", (long long)max_records);
        } else if (len > 0 && text_h[i] != ';') {
            const uint8_t *src = text_h + i;
            int64_t dropped = 0;
            if (memchr(src, ' ', (size_t)len) || memchr(src, '\t', (size_t)len) || memchr(src, '\r', (size_t)len))
                for (int64_t q = 0; q < len; ++q) dropped += src[q] == ' ' || src[q] == '\t' || src[q] == '\r';
            const int64_t kept = len - dropped;
            if (kept > 0) {
                if (!open_record)
                    DNATOK_REQUIRE(begin_record(0, 0), DNATOK_E_TOO_LARGE,
                                   "dnatok_host_fasta_scan: more than %lld records", (long long)max_records);
                if (writing) {
                    DNATOK_REQUIRE(bases + kept <= seq_capacity, DNATOK_E_TOO_LARGE,
                                   "dnatok_host_fasta_scan: more than %lld bases", (long long)seq_capacity);
                    uint8_t *dst = seq_out + bases;
                    if (dropped == 0) {
                        memcpy(dst, src, (size_t)len);
                    } else {
                        int64_t w = 0;
                        for (int64_t q = 0; q < len; ++q)
                            if (src[q] != ' ' && src[q] != '\t' && src[q] != '\r') dst[w++] = src[q];
                    }
                    if (upper_case)
                        for (int64_t q = 0; q < kept; ++q) dst[q] = (uint8_t)(dst[q] - ((dst[q] >= 'a' && dst[q] <= 'z') ? 32 : 0));
                }
                bases += kept;
            }
        }
        i = e + 1;
    }
    if (writing) offsets_out[rec] = bases;
    *n_records = rec;
    *n_bases = bases;
    return DNATOK_OK;
}
