/*
 * dnatok_hip.h -- C ABI of libdnatok_hip.so, the MI355X (gfx950) DNA tokenization backend.
 *
 * Plain pointers and sizes only; no torch / pybind types.  Unless marked "host", every
 * pointer is a DEVICE pointer the caller owns.  `stream` is a hipStream_t passed as void*
 * (NULL = the default stream).  Every launch is asynchronous on that stream and nothing
 * here synchronises the device.  Functions return 0 on success or a negative DNATOK_E_*
 * code; dnatok_last_error() gives the message of the calling thread's last failure.
 *
 * Each entry point names the interface of the reference (eniktab/DNAtok, paths relative
 * to its root) that it stands in for.
 */
#ifndef DNATOK_HIP_H
#define DNATOK_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define DNATOK_VERSION 100

#define DNATOK_OK            0
#define DNATOK_E_INVALID    -1   /* bad argument */
#define DNATOK_E_HIP        -2   /* a HIP runtime call failed */
#define DNATOK_E_TOO_LARGE  -3   /* vocabulary / merge table / input beyond what the kernels index */
#define DNATOK_E_SCRATCH    -4   /* scratch buffer too small */

/* per-row status bits written by the k-mer encoder */
#define DNATOK_ROW_INVALID_BYTE  1   /* a byte outside the digit table (encoded as N) */
#define DNATOK_ROW_MISSING_KMER  2   /* a window with neither an id nor an expansion */
#define DNATOK_ROW_TRUNCATED     4   /* more tokens than the row stride holds */

typedef struct dnatok_char_table dnatok_char_t;
typedef struct dnatok_kmer_table dnatok_kmer_t;
typedef struct dnatok_bpe_table  dnatok_bpe_t;

int         dnatok_version(void);
const char *dnatok_last_error(void);

/* ---------------------------------------------------------------------------------------
 * Single-nucleotide (char) encoder.
 * Replaces DNATok._encode_batch_ascii_lut_numpy / _variable_length
 * (src/dna_tokenizer.py:1779-1858), DNATok._encode_batch_numpy's first-column fix-up
 * (1582-1589) and DNATok._map_ascii_bytes_to_ids_cuda (2653-2723).
 * ------------------------------------------------------------------------------------- */

/* lut_h / start_lut_h: host int32[256]; start_lut_h may be NULL (no separate table for the
 * first character of a row). */
int  dnatok_char_table_create(const int32_t *lut_h, const int32_t *start_lut_h, int32_t pad_id,
                              dnatok_char_t **out);
void dnatok_char_table_destroy(dnatok_char_t *t);

/* Ragged rows -> ids int32[n_rows, t_out] and mask uint8[n_rows, t_out] (mask may be NULL).
 * Row b is bytes[offsets[b] .. offsets[b+1]); rows longer than t_out are cut, shorter ones
 * padded with pad_id on the right (pad_left = 0) or on the left (pad_left = 1). */
int dnatok_char_encode_padded(const dnatok_char_t *t, const uint8_t *bytes, const int64_t *offsets,
                              int64_t n_rows, int64_t t_out, int pad_left,
                              int32_t *ids, uint8_t *mask, void *stream);

/* The same with ids of id_bytes-wide integers (1: uint8, 2: int16, 4: int32, 8: int64; an id that
 * does not fit is cut to the width): what DNATok.encode_batch_with_padding returns once it has
 * narrowed its ids to the smallest type that holds the vocabulary (src/dna_tokenizer.py:2150-2236),
 * written directly in that type, padded on either side, at any width t_out (a fixed token_len, a
 * multiple of pad_multiple). */
int dnatok_char_encode_padded_as(const dnatok_char_t *t, const uint8_t *bytes, const int64_t *offsets,
                                 int64_t n_rows, int64_t t_out, int pad_left,
                                 void *ids, int32_t id_bytes, uint8_t *mask, void *stream);

/* Flat stream: ids[i] = lut[bytes[i]], i < total; mask (may be NULL) is set to 1.
 * row_len > 0 declares equal-length rows, so that positions i % row_len == 0 use the start
 * table; row_len = 0 means no row structure.  This is also the dense [B, T] -> [B, T] case. */
int dnatok_char_encode_packed(const dnatok_char_t *t, const uint8_t *bytes, int64_t total,
                              int64_t row_len, int32_t *ids, uint8_t *mask, void *stream);

/* Fused tokenize + embedding gather: out[i, :] = emb[lut[bytes[i]], :] for i < total, without the
 * id tensor in between.  Replaces DNATok._fused_tokenize_gather (src/dna_tokenizer.py:3465-3532,
 * a Triton kernel there).  emb is [n_vocab] rows of row_bytes bytes each (any element type; rows
 * and output 16-byte aligned, row_bytes a multiple of 16), out is [total] rows of row_bytes.
 * An id outside [0, n_vocab) gives a row of zeros.  row_len as in dnatok_char_encode_packed. */
int dnatok_char_embed_packed(const dnatok_char_t *t, const uint8_t *bytes, int64_t total,
                             int64_t row_len, const void *emb, int32_t n_vocab, int64_t row_bytes,
                             void *out, void *stream);

/* 2-bit packed bases -> ids.  packed is uint8[n_rows, ceil(row_len / 4)] on the device: four bases
 * per byte, the first in the low two bits, codes A C G T = 0 1 2 3 (what dnatok_host_pack_2bit
 * writes).  ids is [n_rows, row_len] of id_bytes-wide integers (1: uint8, 4: int32, 8: int64);
 * ids[b, t] = lut["ACGT"[code]], column 0 from the start table when the table has one.  Replaces
 * DNATok._unpack_2bit_to_ids_cuda / _unpack_2bit_to_ids_cuda_u8 (src/dna_tokenizer.py:3212-3330). */
int dnatok_char_unpack_2bit(const dnatok_char_t *t, const uint8_t *packed, int64_t n_rows,
                            int64_t row_len, void *ids, int32_t id_bytes, void *stream);

/* ---------------------------------------------------------------------------------------
 * Host-side ingest (CPU code, host pointers, no device work).
 * ------------------------------------------------------------------------------------- */

/* In place: a-z -> A-Z when upper_case; then, when invalid_to_n, every byte outside ACGTN (outside
 * ACGTNacgtn when upper_case = 0) becomes 'N'.  *n_replaced (may be NULL) counts those.  Replaces the
 * numpy passes of DNATok._encode_ascii_bytes_impl (src/dna_tokenizer.py:2637-2649). */
int dnatok_host_clean_ascii(uint8_t *bytes_h, int64_t n, int upper_case, int invalid_to_n,
                            int64_t *n_replaced);

/* ASCII rows uint8[n_rows, row_len] -> packed uint8[n_rows, ceil(row_len / 4)]:
 * byte = c0 | c1 << 2 | c2 << 4 | c3 << 6 with A C G T (either case) = 0 1 2 3 and every other byte,
 * N included, 0; the last byte of a row is filled with 0 codes.  Replaces
 * DNATok.encode_batch_to_packed_2bit (src/dna_tokenizer.py:3143-3210). */
int dnatok_host_pack_2bit(const uint8_t *ascii_h, int64_t n_rows, int64_t row_len, uint8_t *packed_h);

/* FASTA text (n bytes in host memory, e.g. a memory-mapped file) -> the sequences of all records laid
 * end to end in seq_out, offsets_out[n_records + 1] (the layout every encoder here takes) and, when
 * name_spans_out is not NULL, the byte span [lo, hi) of each record's header line in the text (without
 * the '>').  Line ends, blanks and tabs inside sequence lines are dropped, lines that start with ';'
 * are skipped, bases in front of the first header form a record of their own (name span 0, 0),
 * a-z -> A-Z when upper_case.  Called with seq_out = NULL it only counts: *n_records and *n_bases are
 * the sizes the second call needs (seq_capacity bases, max_records records).  The reference has no
 * reader of its own: its callers bring Python strings (src/dna_tokenizer.py:2594-2651, one
 * str.encode per row); this is the same hand-over for callers that start from a file. */
int dnatok_host_fasta_scan(const uint8_t *text_h, int64_t n, int upper_case, uint8_t *seq_out,
                           int64_t seq_capacity, int64_t *offsets_out, int64_t *name_spans_out,
                           int64_t max_records, int64_t *n_records, int64_t *n_bases);

/* ---------------------------------------------------------------------------------------
 * Non-overlapping k-mer encoder (grid-aligned windows, per-window fallback, tail as single
 * characters).  Replaces DNATok._encode_batch_kmer_numpy_partial (src/dna_tokenizer.py:
 * 1369-1474), _encode_kmer_fallback_from_lut / _merge_kmer_fallback (1896-2047) and
 * _map_kmer_bytes_to_ids_cuda / _expand_kmer_packed_cuda (2736-2940); the tables are the
 * ones DNATok._build_kmer_lut (743-822) produces.
 * ------------------------------------------------------------------------------------- */

/* All table arguments are host pointers.
 *   digit_h[256]     base-5 digit of a byte (A0 C1 G2 T3 N4), -1 = not in the alphabet
 *   kmer_lut_h[5^k]  token id of a window (digits most significant first), or -1
 *   exp_off_h/exp_len_h[5^k], exp_flat_h[n_flat]  token list of a window whose id is -1
 *                    (may all be NULL / 0: then such windows emit missing_id)
 *   single_h[256]    token id of one character (used for the trailing len % k bases)
 * 2 <= k <= 8. */
int  dnatok_kmer_table_create(int k, const int8_t *digit_h, const int32_t *kmer_lut_h,
                              const int32_t *exp_off_h, const int32_t *exp_len_h,
                              const int32_t *exp_flat_h, int64_t n_flat,
                              const int32_t *single_h, int32_t pad_id, int32_t missing_id,
                              dnatok_kmer_t **out);
void dnatok_kmer_table_destroy(dnatok_kmer_t *t);

/* TEST AND MEASUREMENT ONLY (no counterpart in the reference; results are identical either way).
 * Which of the two k-mer kernels the calls with this table use.  A batch of up to max_rows rows is
 * encoded with a workgroup per row (four waves share a row: the latency of a small batch), a
 * larger one with a wave per row (the bandwidth of a large one).  -1 (default): as many rows as
 * workgroups fit the chip at once; 0: always a wave per row (and no split by row class in
 * dnatok_kmer_encode_padded_sized).  The setting belongs to the table object; a call reads it once
 * when it starts. */
int dnatok_kmer_table_set_team_rows(dnatok_kmer_t *t, int32_t max_rows);

/* ids int32[n_rows, t_cap], mask uint8[n_rows, t_cap] (NULL allowed): t_cap is the row stride.
 * lengths int32[n_rows] receives each row's token count (also when it exceeds t_cap),
 * status int32[n_rows] the DNATOK_ROW_* bits (NULL allowed), max_len int32[1] the largest
 * stored row length (NULL allowed).
 * fill_to > 0: every row is padded to column fill_to (<= t_cap).
 * fill_to = 0: rows are padded to the longest row of the batch, found on the device, so the
 *              caller may view ids[:, :max_len] without a second pass over the data.
 * fill_to < 0: as fill_to = 0, with -fill_to as the caller's guess of that longest row (say,
 *              the width of the previous batch of a stream).  Rows are padded to the guess while
 *              they are written and only what is missing afterwards; a guess that is too small
 *              or too large costs time, never correctness (cells past max_len are unspecified).
 * Calls on one table may overlap on different streams (fill_to <= 0 keeps its running maximum in
 * a device word per stream); calls issued from several host threads are serialised only for the
 * moment that word is looked up. */
int dnatok_kmer_encode_padded(const dnatok_kmer_t *t, const uint8_t *bytes, const int64_t *offsets,
                              int64_t n_rows, int64_t t_cap, int64_t fill_to,
                              int32_t *ids, uint8_t *mask, int32_t *lengths, int32_t *status,
                              int32_t *max_len, void *stream);

/* The same for a caller that knows the batch's size in bytes (`total`; the strings' lengths are on
 * the host anyway), which tells the call how long the rows are on average.  The reference groups the
 * rows of a batch by length before it encodes them (src/dna_tokenizer.py:1476-1531); here a batch
 * of mostly short rows with some long ones among them (mean at most 384 windows, stride above 384
 * cells) is split between two kernels over the one output: the rows of at most 384 units get
 * sixteen lanes each, the others a wave each, chosen row by row on the device from the offsets.
 * Any other batch is encoded exactly as by dnatok_kmer_encode_padded.  Results are identical. */
int dnatok_kmer_encode_padded_sized(const dnatok_kmer_t *t, const uint8_t *bytes, const int64_t *offsets,
                                    int64_t n_rows, int64_t total, int64_t t_cap, int64_t fill_to,
                                    int32_t *ids, uint8_t *mask, int32_t *lengths, int32_t *status,
                                    int32_t *max_len, void *stream);

/* Packed layout, for ragged batches whose padded form would be mostly padding (100,000 reads of
 * 100-300 bp beside a few rows of 20 kbp): ids_out int32[sum of lengths] holds the rows' tokens
 * back to back, out_offsets int64[n_rows + 1] their boundaries, mask_out uint8 (NULL allowed) is
 * one per token, lengths / status as above.  ids_out and mask_out have room for `total` cells (a row
 * never has more tokens than bytes).  Two passes over the bytes: the rows' token counts, their
 * prefix sum, then the tokens; no padding is written and nothing returns to the host.  The k-mer
 * counterpart of dnatok_pack_ragged; the reference has no packed k-mer output (its rows go through
 * _pad_id_list, src/dna_tokenizer.py:1878-1894). */
int dnatok_kmer_encode_packed(const dnatok_kmer_t *t, const uint8_t *bytes, const int64_t *offsets,
                              int64_t n_rows, int64_t total, int32_t *ids_out, int64_t *out_offsets,
                              uint8_t *mask_out, int32_t *lengths, int32_t *status, void *stream);

/* ---------------------------------------------------------------------------------------
 * BPE merge engine.  Replaces the pybind class DNATokBPE and its kernel
 * (src/dnatok_bpe_kernel/dnatok_bpe.cu:237-740 bpe_kernel, 761-791 build_vocab_from_merges,
 * 797-838 constructor, 865-947 tokenize_batch, 956-1015 ensure_workspace).
 * ------------------------------------------------------------------------------------- */

/* Host arrays.  Merge rule i (its rank) is (pair_a_h[i], pair_b_h[i]) -> new_id_h[i]; ids are
 * symbol indices < n_symbols (the reference's kernel id space: 0..255 bytes, then merge
 * results in first-seen order).  byte_to_id_h[256] gives the initial symbol of a byte.
 * out_remap_h[n_symbols] (may be NULL) translates a symbol to the id that is written out,
 * which is what GPUTokBPEBackend's remap table does after the kernel
 * (src/gputok_bpe_backend.py:451-466, 581).  n_symbols <= 65535, n_merges <= 65534. */
int  dnatok_bpe_table_create(const int32_t *byte_to_id_h, const int32_t *pair_a_h,
                             const int32_t *pair_b_h, const int32_t *new_id_h, int32_t n_merges,
                             int32_t n_symbols, const int32_t *out_remap_h, dnatok_bpe_t **out);
void dnatok_bpe_table_destroy(dnatok_bpe_t *t);

/* Bytes of device scratch dnatok_bpe_encode needs for a batch whose longest row has max_len
 * bytes and whose rows sum to total bytes. */
size_t dnatok_bpe_scratch_bytes(const dnatok_bpe_t *t, int64_t n_rows, int64_t max_len,
                                int64_t total);

/* Row b's tokens are written to tok_tmp[offsets[b] .. offsets[b] + lengths[b]) (a row never has
 * more tokens than bytes), tok_tmp is int32[total].  max_len is a host-known upper bound of the
 * row lengths (it selects the kernel variant); scratch is device memory of at least
 * dnatok_bpe_scratch_bytes() bytes, reusable across calls on the same stream. */
int dnatok_bpe_encode(const dnatok_bpe_t *t, const uint8_t *bytes, const int64_t *offsets,
                      int64_t n_rows, int64_t max_len, int64_t total,
                      void *scratch, size_t scratch_bytes,
                      int32_t *tok_tmp, int32_t *lengths, void *stream);

/* dnatok_bpe_encode that also writes the single-character ids of the same bytes, in the same pass
 * over them: char_ids[i] = char_lut[bytes[i]] for every byte of every row (int32[total], laid out as
 * the bytes are: row b at offsets[b]), char_mask[i] = 1 (uint8[total], NULL allowed); char_lut is a
 * device int32[256].  This is dnatok_char_encode_packed fused into the merge engine for batches that
 * go through both tokenizers (the reference runs the two one after the other: the ASCII table
 * path, src/dna_tokenizer.py:2594-2651, and GPUTokBPEBackend.encode_batch,
 * src/gputok_bpe_backend.py:531-601); tokens, lengths, scratch and errors as for dnatok_bpe_encode. */
int dnatok_bpe_encode_with_chars(const dnatok_bpe_t *t, const uint8_t *bytes, const int64_t *offsets,
                                 int64_t n_rows, int64_t max_len, int64_t total,
                                 void *scratch, size_t scratch_bytes,
                                 int32_t *tok_tmp, int32_t *lengths,
                                 const int32_t *char_lut, int32_t *char_ids, uint8_t *char_mask,
                                 void *stream);

/* dnatok_bpe_encode and dnatok_pad_rows in one pass: row b's ids go straight to ids[b * stride ..]
 * (int32[n_rows, stride]), through remap (kernel id -> tokenizer id, NULL: none), pad_id behind them
 * up to the stride, mask (uint8[n_rows, stride], NULL allowed) 1 for a token and 0 for padding.  This
 * is the tail of GPUTokBPEBackend.encode_batch (the remap LUT and the [B, T_max] padding,
 * src/gputok_bpe_backend.py:624-638, 660-674) done by the merge engine while it writes a row's
 * tokens out: no token run in memory in between, no second launch.  lengths[b] receives the row's
 * full token count and *longest (device int32[1]; NULL: the caller takes it from the lengths, and
 * the call ends a few microseconds earlier) the largest of them: a row with more tokens than
 * the stride keeps its first `stride`, so a caller that sized the stride by a guess compares
 * the longest row with it and, when that is larger, calls again with a stride of at least that (a row
 * never has more tokens than bytes).  Rows of at most dnatok_bpe_padded_direct_max() bytes are
 * written this way; a batch with a longer row (max_len above it) is assembled in tok_tmp
 * (int32[total], NULL allowed otherwise) and padded from there by the kernels of the two calls.
 * scratch, max_len and errors as for dnatok_bpe_encode. */
int dnatok_bpe_encode_padded(const dnatok_bpe_t *t, const uint8_t *bytes, const int64_t *offsets,
                             int64_t n_rows, int64_t max_len, int64_t total,
                             void *scratch, size_t scratch_bytes, int32_t *tok_tmp,
                             const int32_t *remap, int32_t pad_id, int64_t stride,
                             int32_t *ids, uint8_t *mask, int32_t *lengths, int32_t *longest,
                             void *stream);

/* The same with the two layout choices DNATok and GPUTokBPEBackend make after the encode, so that
 * the engine's launch writes the final tensor: ids = [n_rows, stride] of id_bytes-wide integers
 * (1: uint8, 2: int16, 4: int32, 8: int64 -- the reference's backend returns int64,
 * src/gputok_bpe_backend.py:581-600; DNATok.encode_batch_with_padding the narrowest type that holds
 * the vocabulary, src/dna_tokenizer.py:2150-2236), and pad_left = 1 puts a row's tokens at the END
 * of its `stride` cells with the padding before them (src/dna_tokenizer.py:2072-2078 re-pads the
 * backend's rows to padding_side): the caller views the last `width` columns.  A row with more tokens
 * than the stride keeps its first `stride` either way. */
int dnatok_bpe_encode_padded_as(const dnatok_bpe_t *t, const uint8_t *bytes, const int64_t *offsets,
                                int64_t n_rows, int64_t max_len, int64_t total,
                                void *scratch, size_t scratch_bytes, int32_t *tok_tmp,
                                const int32_t *remap, int32_t pad_id, int64_t stride, int pad_left,
                                void *ids, int32_t id_bytes, uint8_t *mask, int32_t *lengths,
                                int32_t *longest, void *stream);

/* Longest row, in bytes, that dnatok_bpe_encode_padded writes without tok_tmp with this table
 * (the size of an extended chunk, 2048 unless dnatok_bpe_table_set_chunk_geometry changed it;
 * t = NULL: the shipped value). */
int64_t dnatok_bpe_padded_direct_max(const dnatok_bpe_t *t);

/* The same encode for callers that cannot allocate device memory or hand over a work buffer: code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has no
 * counterpart in the reference (whose tokenize_batch grows torch tensors on demand,
 * src/dnatok_bpe_kernel/dnatok_bpe.cu:956-1015).  The work space is an array of
 * DNATOK_BPE_STATIC_SCRATCH_BYTES bytes inside the library's own device image, one copy per GPU,
 * held until the process ends; the call allocates and frees nothing.  A batch that needs more
 * (dnatok_bpe_scratch_bytes grows with the row count, the number of 1792-byte chunks of the rows
 * above 2048 bytes, and the longest row) is refused with DNATOK_E_TOO_LARGE; rows that have to be
 * redone whole are then redone fewer at a time before that happens.  All calls on one GPU share
 * the array: two calls whose device work overlaps (different streams, or another thread) race;
 * calls on one stream, and replays of a captured call, are fine.  Before a call is captured, one
 * eager call of the same shape class (row count, longest row, total of the same order) must have
 * run in the process: the first call of each kernel form asks the runtime for the form's
 * attributes and residency, which a capture does not allow.  Inputs, outputs and results as for
 * dnatok_bpe_encode. */
#define DNATOK_BPE_STATIC_SCRATCH_BYTES (32u << 20)
size_t dnatok_bpe_static_scratch_bytes(void);
int dnatok_bpe_encode_static(const dnatok_bpe_t *t, const uint8_t *bytes, const int64_t *offsets,
                             int64_t n_rows, int64_t max_len, int64_t total,
                             int32_t *tok_tmp, int32_t *lengths, void *stream);

/* TEST ONLY, no counterpart in the reference: the geometry the calls with this table cut rows
 * longer than core + 2 * overlap bytes with: chunks of `core` bytes, extended by `overlap` bytes on
 * both sides, joined at seams inside the overlaps.  The shipped geometry is (1792, 128); (0, 0)
 * restores it.  Tests pass small chunks so that rows of a few kilobytes go through thousands of
 * seams and whole-row fallbacks.  Results never depend on the geometry.  The setting belongs to the
 * table object; a call reads it once when it starts (size the scratch buffer after setting it). */
int dnatok_bpe_table_set_chunk_geometry(dnatok_bpe_t *t, int32_t core, int32_t overlap);

/* MEASUREMENT ONLY: where the merge table of the calls with this table object is kept (no
 * counterpart in the reference, whose kernel reads its hash table from global memory,
 * dnatok_bpe.cu:822-837).  A table of at most 8192 symbols and 4095 rules also has a compact form
 * of 48 KB.  mode 0 (default): every batch reads the table from global memory (L2), which measured
 * faster.  mode 1: a batch of rows of at most 1024 bytes, few enough for one row per resident
 * workgroup with those 48 KB added to each, is encoded by workgroups that keep the compact form in
 * LDS.  mode 2: the compact form for every batch of rows of at most 1024 bytes that one launch
 * encodes whole.  Results are identical in all modes. */
int dnatok_bpe_table_set_placement(dnatok_bpe_t *t, int32_t mode);

/* ---------------------------------------------------------------------------------------
 * Ragged-batch packer: turns per-row token runs (tok_tmp + in_offsets + lengths, as the BPE
 * engine leaves them) into the tensors a model consumes, without a host round trip.
 * Replaces the torch op chain of GPUTokBPEBackend.encode_batch
 * (src/gputok_bpe_backend.py:578-601: remap gather, lens.max().item(), arange mask, where).
 * ------------------------------------------------------------------------------------- */

/* Packed layout: ids_out int32[sum lengths] holds the rows back to back, out_offsets
 * int64[n_rows + 1] their boundaries, mask_out uint8[sum lengths] (NULL allowed) is all ones.
 * remap (device int32, NULL allowed) translates every id. */
int dnatok_pack_ragged(const int32_t *tok_tmp, const int64_t *in_offsets, const int32_t *lengths,
                       int64_t n_rows, const int32_t *remap, int32_t *ids_out,
                       int64_t *out_offsets, uint8_t *mask_out, void *stream);

/* Padded layout: ids int32[n_rows, t_cap] / mask uint8[n_rows, t_cap]; fill_to and max_len as
 * for dnatok_kmer_encode_padded. */
int dnatok_pad_rows(const int32_t *tok_tmp, const int64_t *in_offsets, const int32_t *lengths,
                    int64_t n_rows, const int32_t *remap, int32_t pad_id, int64_t t_cap,
                    int64_t fill_to, int32_t *ids, uint8_t *mask, int32_t *max_len, void *stream);

/* The same with everything DNATok.encode_batch_to_ids / encode_batch_with_padding do to token rows
 * after the encode (src/dna_tokenizer.py:1878-1894 _pad_id_list: padding side and token_len;
 * 2150-2236: pad_multiple and the narrowest id type), in the one launch:
 *   width     = fill_to, or with fill_to = 0 the longest row; then at least min_width, rounded up
 *               to a multiple of pad_multiple (0 or 1: none), at most t_cap; written to width_out
 *               (int32[1], NULL allowed), while max_len still receives the longest row;
 *   pad_left  = 1: a row's tokens end at column width - 1 (a row longer than the width keeps its
 *               first `width` tokens), 0: they start at column 0;
 *   ids       = [n_rows, t_cap] of id_bytes-wide integers (1: uint8, 2: int16, 4: int32, 8: int64). */
int dnatok_pad_rows_as(const int32_t *tok_tmp, const int64_t *in_offsets, const int32_t *lengths,
                       int64_t n_rows, const int32_t *remap, int32_t pad_id, int64_t t_cap,
                       int64_t fill_to, int64_t min_width, int64_t pad_multiple, int pad_left,
                       void *ids, int32_t id_bytes, uint8_t *mask, int32_t *max_len,
                       int32_t *width_out, void *stream);

/* ---------------------------------------------------------------------------------------
 * Tokenizer normalizer on the device: the steps GPUTokBPEBackend compiles from a
 * tokenizer.json "normalizer" and applies string by string on the host before the kernel
 * (_compile_normalizer_step / _compile_normalizer, src/gputok_bpe_backend.py:179-248; applied at
 * 531-535), here applied to the ragged rows of bytes already on the device.
 * ------------------------------------------------------------------------------------- */

#define DNATOK_NORM_MAX_BYTES   16   /* longest pattern / replacement / prefix of a step */

#define DNATOK_NORM_STRIP        1   /* flags bit 0: left, bit 1: right; ASCII whitespace as str.strip() */
#define DNATOK_NORM_REPLACE      2   /* every occurrence of pattern -> content (str.replace); the pattern
                                        must not overlap itself (no proper prefix equal to a suffix) */
#define DNATOK_NORM_REPLACE_RUN  3   /* every maximal run of the byte pattern[0] that is at least `flags`
                                        long -> one content (the regex  c{n,}  with n = flags, 1..64) */
#define DNATOK_NORM_PREPEND      4   /* content in front of every row, empty rows included */
#define DNATOK_NORM_LOWERCASE    5   /* A-Z -> a-z */

typedef struct dnatok_norm_step {
    int32_t kind;
    int32_t flags;
    int32_t pattern_len;
    int32_t content_len;
    uint8_t pattern[DNATOK_NORM_MAX_BYTES];
    uint8_t content[DNATOK_NORM_MAX_BYTES];
} dnatok_norm_step;

/* Host-side arithmetic (steps_h is a host array): upper bounds of the total bytes and of the
 * longest row after the steps, for a batch of n_rows rows of `total` bytes whose longest row has
 * max_len bytes, and the bytes of device scratch dnatok_normalize_rows needs.  Also validates the
 * steps.  Any of the three outputs may be NULL. */
int dnatok_normalize_bounds(const dnatok_norm_step *steps_h, int32_t n_steps, int64_t n_rows,
                            int64_t total, int64_t max_len, int64_t *out_total, int64_t *out_max_len,
                            size_t *scratch_bytes);

/* Applies the steps in order to rows bytes[offsets[b] .. offsets[b+1]) (offsets[0] = 0,
 * offsets[n_rows] = total) and writes the rows back to back into out_bytes (capacity at least the
 * out_total bound) with their boundaries in out_offsets int64[n_rows + 1].  The input is left
 * untouched; sizes after the first step exist only on the device, so nothing is read back. */
int dnatok_normalize_rows(const dnatok_norm_step *steps_h, int32_t n_steps, const uint8_t *bytes,
                          const int64_t *offsets, int64_t n_rows, int64_t total, int64_t max_len,
                          uint8_t *out_bytes, int64_t out_capacity, int64_t *out_offsets,
                          void *scratch, size_t scratch_bytes, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* DNATOK_HIP_H */
