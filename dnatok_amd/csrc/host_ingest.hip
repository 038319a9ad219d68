// Host-side ingest helpers: what a caller does to its strings before the bytes cross PCIe.
// Plain CPU code (no device work): one pass over the bytes instead of one numpy pass per rule.
#include "common.hpp"

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
