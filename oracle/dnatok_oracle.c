/*
 * dnatok_oracle.c -- CPU restatement of the DNA tokenization hot path.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the checker the HIP kernels are
 * compared against; nothing on the product path may call it.  Only tests/,
 * __graft_entry__.smoke() and bench.py's cpu_baseline leg load it.
 *
 * What each function restates (reference = eniktab/DNAtok, paths relative to
 * its root; HF = Hugging Face `tokenizers`, pinned by the reference at
 * tokenizers==0.22.1 in docker/requirements.txt:13, whose Rust source is not
 * part of the reference tree -- its published BPE word-merge algorithm is
 * restated from the library's documented behaviour):
 *
 *   oracle_char_encode_padded / _packed
 *       ids[b,t] = lut[byte[b,t]], first column optionally from a start table,
 *       right- or left-padded with the pad id, mask = 1 on real tokens.
 *       src/dna_tokenizer.py:1779-1858 (numpy path), 2653-2723 (device path),
 *       mask: src/gputok_bpe_backend.py:593-600.
 *   oracle_kmer_encode_row
 *       base-5 digits (A0 C1 G2 T3 N4) -> window code -> kmer_lut; a window
 *       whose entry is -1 expands to its own token list; the trailing
 *       len % k bases go through the single-character table.
 *       src/dna_tokenizer.py:743-822 (tables), 1369-1474 (grid-aligned
 *       windows + tail), 1896-1953 (per-window expansion).
 *   oracle_bpe_encode_row
 *       HF BPE word merge: every adjacent pair that has a merge rule enters a
 *       min-heap keyed (rank, position); pop, skip stale entries, merge,
 *       push the two new neighbour pairs.  Same result as "apply the
 *       lowest-rank rule at its leftmost occurrence, repeat"
 *       (src/dnatok_bpe_kernel/dnatok_bpe.cu:3-5, 172-176).
 *   oracle_bpe_encode_row_naive
 *       the textbook O(n^2) form of the same rule, kept to pin the heap form.
 *
 * Pinned by tests/test_oracle.py against the installed HF `tokenizers`
 * library (WordLevel char / 6-mer tokenizers and the BpeTrainer-trained
 * vocabularies), against closed forms, and heap-vs-naive on random input.
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------ char */

void oracle_char_encode_padded(const int32_t *lut, const int32_t *start_lut, int32_t pad_id,
                               const uint8_t *bytes, const int64_t *offsets, int64_t n_rows,
                               int64_t t_out, int pad_left, int32_t *ids, uint8_t *mask)
{
    for (int64_t b = 0; b < n_rows; ++b) {
        const uint8_t *row = bytes + offsets[b];
        int64_t len = offsets[b + 1] - offsets[b];
        if (len > t_out) len = t_out;
        int64_t shift = pad_left ? (t_out - len) : 0;
        int32_t *o = ids + b * t_out;
        uint8_t *m = mask ? mask + b * t_out : NULL;
        for (int64_t j = 0; j < t_out; ++j) {
            o[j] = pad_id;
            if (m) m[j] = 0;
        }
        for (int64_t j = 0; j < len; ++j) {
            const int32_t *tab = (j == 0 && start_lut) ? start_lut : lut;
            o[shift + j] = tab[row[j]];
            if (m) m[shift + j] = 1;
        }
    }
}

void oracle_char_encode_packed(const int32_t *lut, const uint8_t *bytes, int64_t total,
                               int32_t *ids)
{
    for (int64_t i = 0; i < total; ++i) ids[i] = lut[bytes[i]];
}

/* ----------------------------------------------------------------- k-mer */

/*
 * digit[256]   : base-5 digit of a byte (0..4), or -1 for a byte outside the alphabet
 *                (treated as N, digit 4, and reported through *status bit 0).
 * kmer_lut[5^k]: token id of a window, or -1.
 * exp_off/exp_len/exp_flat: token list of a window whose kmer_lut entry is -1
 *                (exp_len 0 = no expansion known: missing_id is emitted and
 *                *status bit 1 is set).
 * single[256]  : token id of one character, used for the trailing len % k bases.
 * Returns the number of tokens the row produces; at most `cap` are stored.
 */
int64_t oracle_kmer_encode_row(int k, const int8_t *digit, const int32_t *kmer_lut,
                               const int32_t *exp_off, const int32_t *exp_len,
                               const int32_t *exp_flat, const int32_t *single,
                               int32_t missing_id, const uint8_t *row, int64_t len,
                               int32_t *out, int64_t cap, int32_t *status)
{
    int64_t n = 0;
    int64_t full = len / k;
    int32_t st = 0;
    for (int64_t w = 0; w < full; ++w) {
        int64_t code = 0;
        for (int i = 0; i < k; ++i) {
            int d = digit[row[w * k + i]];
            if (d < 0) { d = 4; st |= 1; }
            code = code * 5 + d;
        }
        int32_t id = kmer_lut[code];
        if (id >= 0) {
            if (n < cap) out[n] = id;
            ++n;
        } else if (exp_len && exp_len[code] > 0) {
            for (int32_t e = 0; e < exp_len[code]; ++e) {
                if (n < cap) out[n] = exp_flat[exp_off[code] + e];
                ++n;
            }
        } else {
            st |= 2;
            if (n < cap) out[n] = missing_id;
            ++n;
        }
    }
    for (int64_t j = full * k; j < len; ++j) {
        if (n < cap) out[n] = single[row[j]];
        ++n;
    }
    if (status) *status = st;
    return n;
}

/* Whole batch into a padded [n_rows, t_cap] matrix (ids + mask), rows padded to t_cap. */
void oracle_kmer_encode_batch(int k, const int8_t *digit, const int32_t *kmer_lut,
                              const int32_t *exp_off, const int32_t *exp_len,
                              const int32_t *exp_flat, const int32_t *single,
                              int32_t missing_id, int32_t pad_id, const uint8_t *bytes,
                              const int64_t *offsets, int64_t n_rows, int64_t t_cap,
                              int32_t *ids, uint8_t *mask, int32_t *lengths)
{
    for (int64_t b = 0; b < n_rows; ++b) {
        int32_t st;
        int32_t *o = ids + b * t_cap;
        int64_t n = oracle_kmer_encode_row(k, digit, kmer_lut, exp_off, exp_len, exp_flat, single,
                                           missing_id, bytes + offsets[b],
                                           offsets[b + 1] - offsets[b], o, t_cap, &st);
        lengths[b] = (int32_t)n;
        if (n > t_cap) n = t_cap;
        for (int64_t j = 0; j < t_cap; ++j) {
            if (j >= n) o[j] = pad_id;
            if (mask) mask[b * t_cap + j] = j < n;
        }
    }
}

/* ------------------------------------------------------------------- BPE */

typedef struct {
    uint64_t *keys;     /* (a << 32) | b, or EMPTY */
    uint32_t *rank;
    int32_t *new_id;
    uint64_t mask;
    int32_t n_merges;
} oracle_bpe_table;

#define ORACLE_EMPTY 0xFFFFFFFFFFFFFFFFull

static inline uint64_t mix64(uint64_t x)
{
    x ^= x >> 33; x *= 0xff51afd7ed558ccdull;
    x ^= x >> 33; x *= 0xc4ceb9fe1a85ec53ull;
    x ^= x >> 33;
    return x;
}

/* Merge rule i: (pair_a[i], pair_b[i]) -> new_id[i], rank i.  A pair listed twice keeps
 * its LAST entry (rank and product): HF collects the merges into a map in list order, so a
 * later entry replaces an earlier one (checked against the library in tests/test_oracle.py). */
oracle_bpe_table *oracle_bpe_table_create(const int32_t *pair_a, const int32_t *pair_b,
                                          const int32_t *new_id, int32_t n_merges)
{
    oracle_bpe_table *t = (oracle_bpe_table *)calloc(1, sizeof(*t));
    uint64_t cap = 64;
    while (cap < (uint64_t)n_merges * 2 + 2) cap <<= 1;
    t->keys = (uint64_t *)malloc(cap * sizeof(uint64_t));
    t->rank = (uint32_t *)malloc(cap * sizeof(uint32_t));
    t->new_id = (int32_t *)malloc(cap * sizeof(int32_t));
    t->mask = cap - 1;
    t->n_merges = n_merges;
    for (uint64_t i = 0; i < cap; ++i) t->keys[i] = ORACLE_EMPTY;
    for (int32_t i = 0; i < n_merges; ++i) {
        uint64_t key = ((uint64_t)(uint32_t)pair_a[i] << 32) | (uint32_t)pair_b[i];
        uint64_t h = mix64(key) & t->mask;
        while (t->keys[h] != ORACLE_EMPTY && t->keys[h] != key) h = (h + 1) & t->mask;
        t->keys[h] = key;
        t->rank[h] = (uint32_t)i;
        t->new_id[h] = new_id[i];
    }
    return t;
}

void oracle_bpe_table_destroy(oracle_bpe_table *t)
{
    if (!t) return;
    free(t->keys); free(t->rank); free(t->new_id); free(t);
}

static inline int table_find(const oracle_bpe_table *t, int32_t a, int32_t b,
                             uint32_t *rank, int32_t *new_id)
{
    uint64_t key = ((uint64_t)(uint32_t)a << 32) | (uint32_t)b;
    uint64_t h = mix64(key) & t->mask;
    while (t->keys[h] != ORACLE_EMPTY) {
        if (t->keys[h] == key) { *rank = t->rank[h]; *new_id = t->new_id[h]; return 1; }
        h = (h + 1) & t->mask;
    }
    return 0;
}

typedef struct { uint32_t rank; int32_t pos; int32_t new_id; } heap_item;

static inline int item_less(heap_item a, heap_item b)
{
    return a.rank < b.rank || (a.rank == b.rank && a.pos < b.pos);
}

static void heap_push(heap_item *h, int64_t *n, heap_item it)
{
    int64_t i = (*n)++;
    while (i > 0) {
        int64_t p = (i - 1) >> 1;
        if (!item_less(it, h[p])) break;
        h[i] = h[p];
        i = p;
    }
    h[i] = it;
}

static heap_item heap_pop(heap_item *h, int64_t *n)
{
    heap_item top = h[0];
    heap_item last = h[--(*n)];
    int64_t i = 0;
    for (;;) {
        int64_t c = 2 * i + 1;
        if (c >= *n) break;
        if (c + 1 < *n && item_less(h[c + 1], h[c])) ++c;
        if (!item_less(h[c], last)) break;
        h[i] = h[c];
        i = c;
    }
    if (*n > 0) h[i] = last;
    return top;
}

/*
 * Encode one word (the whole row: no pre-tokenizer).  byte_to_id maps a raw byte to its
 * initial symbol id.  `out` must hold `len` ids.  Returns the token count.
 */
int64_t oracle_bpe_encode_row(const oracle_bpe_table *t, const int32_t *byte_to_id,
                              const uint8_t *row, int64_t len, int32_t *out)
{
    if (len <= 0) return 0;
    int32_t *sym = (int32_t *)malloc(len * sizeof(int32_t));
    int32_t *prev = (int32_t *)malloc(len * sizeof(int32_t));
    int32_t *next = (int32_t *)malloc(len * sizeof(int32_t));
    uint8_t *dead = (uint8_t *)calloc(len, 1);
    /* every merge pushes at most two entries */
    heap_item *heap = (heap_item *)malloc((size_t)(3 * len + 4) * sizeof(heap_item));
    int64_t hn = 0;
    for (int64_t i = 0; i < len; ++i) {
        sym[i] = byte_to_id[row[i]];
        prev[i] = (int32_t)(i - 1);
        next[i] = (i + 1 < len) ? (int32_t)(i + 1) : -1;
    }
    for (int64_t i = 0; i + 1 < len; ++i) {
        uint32_t r; int32_t nid;
        if (table_find(t, sym[i], sym[i + 1], &r, &nid)) {
            heap_item it = { r, (int32_t)i, nid };
            heap_push(heap, &hn, it);
        }
    }
    while (hn > 0) {
        heap_item top = heap_pop(heap, &hn);
        int32_t p = top.pos;
        if (dead[p]) continue;
        int32_t q = next[p];
        if (q < 0) continue;
        uint32_t r; int32_t nid;
        /* stale entry: the pair standing at p is no longer the one that was queued */
        if (!table_find(t, sym[p], sym[q], &r, &nid) || nid != top.new_id) continue;
        sym[p] = top.new_id;
        dead[q] = 1;
        next[p] = next[q];
        if (next[q] >= 0) prev[next[q]] = p;
        if (prev[p] >= 0 && table_find(t, sym[prev[p]], sym[p], &r, &nid)) {
            heap_item it = { r, prev[p], nid };
            heap_push(heap, &hn, it);
        }
        if (next[p] >= 0 && table_find(t, sym[p], sym[next[p]], &r, &nid)) {
            heap_item it = { r, p, nid };
            heap_push(heap, &hn, it);
        }
    }
    int64_t n = 0;
    for (int32_t i = 0; i >= 0; i = next[i]) out[n++] = sym[i];
    free(sym); free(prev); free(next); free(dead); free(heap);
    return n;
}

/* Textbook form: find the lowest rank over all adjacent pairs, merge its leftmost
 * occurrence, repeat until no pair has a rule. */
int64_t oracle_bpe_encode_row_naive(const oracle_bpe_table *t, const int32_t *byte_to_id,
                                    const uint8_t *row, int64_t len, int32_t *out)
{
    int64_t n = len;
    for (int64_t i = 0; i < len; ++i) out[i] = byte_to_id[row[i]];
    for (;;) {
        uint32_t best = 0xFFFFFFFFu; int64_t at = -1; int32_t best_id = 0;
        for (int64_t i = 0; i + 1 < n; ++i) {
            uint32_t r; int32_t nid;
            if (table_find(t, out[i], out[i + 1], &r, &nid) && r < best) {
                best = r; at = i; best_id = nid;
            }
        }
        if (at < 0) break;
        out[at] = best_id;
        memmove(out + at + 1, out + at + 2, (size_t)(n - at - 2) * sizeof(int32_t));
        --n;
    }
    return n;
}

/* Whole batch, rows independent; tok_tmp[offsets[b] ...] receives row b's tokens. */
void oracle_bpe_encode_batch(const oracle_bpe_table *t, const int32_t *byte_to_id,
                             const uint8_t *bytes, const int64_t *offsets, int64_t n_rows,
                             int32_t *tok_tmp, int32_t *lengths)
{
    for (int64_t b = 0; b < n_rows; ++b)
        lengths[b] = (int32_t)oracle_bpe_encode_row(t, byte_to_id, bytes + offsets[b],
                                                    offsets[b + 1] - offsets[b],
                                                    tok_tmp + offsets[b]);
}
