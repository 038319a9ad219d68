// Ragged-batch packer: per-row token runs -> packed ids + offsets (+mask), or a padded
// [rows, stride] matrix + mask, entirely on the device.  The id remap (kernel id -> tokenizer
// id) is fused into the copy.  One wave copies one row, 64 tokens per step.
#include "common.hpp"

namespace dnatok {

constexpr int kScanThreads = 1024;

// out_offsets[b] = sum of max(lengths[0..b), 0); single workgroup, 4096 rows per step (four
// consecutive rows per thread).  The lengths of kScanSteps steps (32,768 rows) are requested together
// and then scanned step by step out of registers: one trip to memory per 32,768 rows.  (With the
// next step's lengths requested before a step's barrier it was a trip per step, and nothing else
// runs meanwhile: 32,768 rows 20.5 us, now 16.)
constexpr int kScanSteps = 8;

__global__ __launch_bounds__(kScanThreads) void scan_lengths_kernel(
    const int32_t *__restrict__ lengths, int64_t n_rows, int64_t *__restrict__ out_offsets)
{
    constexpr int kPer = 4;
    __shared__ uint32_t wave_tot[2][kScanThreads / 64];
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    int64_t carry = 0;                                   // (every thread keeps the same running total)
    int par = 0;
    for (int64_t base0 = 0; base0 < n_rows; base0 += (int64_t)kScanSteps * kScanThreads * kPer) {
        int32_t v[kScanSteps][kPer];
#pragma unroll
        for (int st = 0; st < kScanSteps; ++st) {
            // (rows beyond the end read the last row and count as 0: no load sits behind a condition)
            const int64_t i0 = base0 + (int64_t)st * kScanThreads * kPer + (int64_t)threadIdx.x * kPer;
#pragma unroll
            for (int q = 0; q < kPer; ++q) v[st][q] = 0;
            if (i0 - (int64_t)threadIdx.x * kPer >= n_rows) continue;      // (no such step: the same for every thread)
#pragma unroll
            for (int q = 0; q < kPer; ++q) {
                const int64_t i = i0 + q;
                const int32_t x = lengths[i < n_rows ? i : n_rows - 1];
                v[st][q] = (i < n_rows && x > 0) ? x : 0;
            }
        }
#pragma unroll
        for (int st = 0; st < kScanSteps; ++st, par ^= 1) {
            const int64_t base = base0 + (int64_t)st * kScanThreads * kPer;
            if (base >= n_rows) break;                   // (the same for every thread)
            const uint32_t mine = (uint32_t)v[st][0] + (uint32_t)v[st][1] + (uint32_t)v[st][2] + (uint32_t)v[st][3];
            const uint32_t inc = wave_inclusive_sum_u32(mine);
            if (lane == 63) wave_tot[par][wv] = inc;
            __syncthreads();                             // (the other half of wave_tot is the previous step's)
            uint32_t before = 0, total = 0;
#pragma unroll
            for (int w = 0; w < kScanThreads / 64; ++w) {
                const uint32_t t = wave_tot[par][w];
                if (w < wv) before += t;
                total += t;
            }
            int64_t at = carry + before + inc - mine;
#pragma unroll
            for (int q = 0; q < kPer; ++q) {
                const int64_t i = base + (int64_t)threadIdx.x * kPer + q;
                if (i < n_rows) out_offsets[i] = at;
                at += v[st][q];
            }
            carry += total;
        }
    }
    if (threadIdx.x == 0) out_offsets[n_rows] = carry;
}

// The same for very many rows (the packed k-mer encode of 100,000 reads: the one workgroup above
// walks them 4096 at a time, a trip to memory per step, 58 us), in two launches of a workgroup per
// tile of 4096 rows: the tiles' sums, then every tile adds up the sums of the tiles before it and
// scans its own rows.
constexpr int kScanTile = kScanThreads * 4;

__device__ __forceinline__ void scan_tile_load(const int32_t *__restrict__ lengths, int64_t n_rows, int64_t base,
                                               uint32_t (&v)[4])
{
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const int64_t i = base + (int64_t)threadIdx.x * 4 + q;
        const int32_t x = i < n_rows ? lengths[i] : 0;
        v[q] = x < 0 ? 0u : (uint32_t)x;
    }
}

__global__ __launch_bounds__(kScanThreads) void scan_tile_sums_kernel(
    const int32_t *__restrict__ lengths, int64_t n_rows, unsigned long long *__restrict__ tile_sum)
{
    __shared__ uint32_t wave_tot[kScanThreads / 64];
    uint32_t v[4];
    scan_tile_load(lengths, n_rows, (int64_t)blockIdx.x * kScanTile, v);
    const uint32_t inc = wave_inclusive_sum_u32(v[0] + v[1] + v[2] + v[3]);
    if ((threadIdx.x & 63) == 63) wave_tot[threadIdx.x >> 6] = inc;
    __syncthreads();
    if (threadIdx.x == 0) {
        unsigned long long t = 0;
        for (int w = 0; w < kScanThreads / 64; ++w) t += wave_tot[w];
        tile_sum[blockIdx.x] = t;
    }
}

__global__ __launch_bounds__(kScanThreads) void scan_tiles_kernel(
    const int32_t *__restrict__ lengths, int64_t n_rows, const unsigned long long *__restrict__ tile_sum,
    int64_t *__restrict__ out_offsets)
{
    __shared__ uint32_t wave_tot[kScanThreads / 64];
    __shared__ unsigned long long part[kScanThreads / 64];
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    uint32_t v[4];
    scan_tile_load(lengths, n_rows, (int64_t)blockIdx.x * kScanTile, v);
    // the tiles before this one
    unsigned long long mine = 0;
    for (unsigned j = threadIdx.x; j < blockIdx.x; j += kScanThreads) mine += tile_sum[j];
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) mine += __shfl_xor(mine, d, 64);
    if (lane == 0) part[wv] = mine;
    const uint32_t own = v[0] + v[1] + v[2] + v[3];
    const uint32_t inc = wave_inclusive_sum_u32(own);
    if (lane == 63) wave_tot[wv] = inc;
    __syncthreads();
    unsigned long long before_tiles = 0;
    uint32_t before = 0, total = 0;
#pragma unroll
    for (int w = 0; w < kScanThreads / 64; ++w) {
        before_tiles += part[w];
        const uint32_t t = wave_tot[w];
        if (w < wv) before += t;
        total += t;
    }
    int64_t at = (int64_t)before_tiles + before + inc - own;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const int64_t i = (int64_t)blockIdx.x * kScanTile + (int64_t)threadIdx.x * 4 + q;
        if (i < n_rows) out_offsets[i] = at;
        at += v[q];
    }
    if (blockIdx.x == gridDim.x - 1 && threadIdx.x == 0) out_offsets[n_rows] = (int64_t)before_tiles + total;
}

// (also used by the packed k-mer encode)  `scratch` (8-byte aligned, NULL allowed) is room the caller
// can spare until the scan is done; with 8 bytes per 4096 rows of it, very many rows take the two
// launches above.
int launch_scan_lengths(const int32_t *lengths, int64_t n_rows, int64_t *out_offsets, void *scratch,
                        size_t scratch_bytes, hipStream_t s)
{
    const int64_t tiles = (n_rows + kScanTile - 1) / kScanTile;
    if (tiles >= 4 && scratch && ((uintptr_t)scratch & 7) == 0 && scratch_bytes >= (size_t)tiles * 8 && tiles < (1 << 20)) {
        scan_tile_sums_kernel<<<(int)tiles, kScanThreads, 0, s>>>(lengths, n_rows, (unsigned long long *)scratch);
        scan_tiles_kernel<<<(int)tiles, kScanThreads, 0, s>>>(lengths, n_rows, (const unsigned long long *)scratch,
                                                             out_offsets);
    } else {
        scan_lengths_kernel<<<1, kScanThreads, 0, s>>>(lengths, n_rows, out_offsets);
    }
    DNATOK_HIP_TRY(hipGetLastError());
    return DNATOK_OK;
}

// output cells one workgroup copies (the grid is 4,096 workgroups whatever the batch, its size being
// known on the device only: with 4,096 cells a batch of 4,096 ragged reads was 1.1 tiles per
// workgroup, i.e. the time of two; 2,048: the call 258.2 -> 255.0 us, eight such batches 1,782 -> 1,786 us;
// 1,024: 256.0 and 1,798 us)
constexpr int kPackTile = 2048;

// Packed layout.  A workgroup takes kPackTile consecutive cells of the packed output, finds the
// first row that reaches into them (binary search in out_offsets) and copies row piece after
// row piece, so that the work per workgroup is the same whether the batch is 4096 short rows
// or a few very long ones.
__global__ __launch_bounds__(256) void pack_copy_kernel(
    const int32_t *__restrict__ tok_tmp, const int64_t *__restrict__ in_offsets, int64_t n_rows,
    const int32_t *__restrict__ remap, const int64_t *__restrict__ out_offsets,
    int32_t *__restrict__ ids_out, uint8_t *__restrict__ mask_out)
{
    const int64_t total = out_offsets[n_rows];
    for (int64_t o0 = (int64_t)blockIdx.x * kPackTile; o0 < total; o0 += (int64_t)gridDim.x * kPackTile) {
        const int64_t o1 = o0 + kPackTile < total ? o0 + kPackTile : total;
        // last row with out_offsets[row] <= o0.  Every wave searches for itself, 64 evenly spaced
        // offsets per step: 4096 rows are two dependent loads instead of the twelve of a binary
        // search (the search is a chain of load latencies at the start of every tile).
        int64_t lo = 0, hi = n_rows;                  // out_offsets[lo] <= o0 < out_offsets[hi] (hi = n_rows: the total)
        while (hi - lo > 1) {
            const int64_t step = (hi - lo + 63) >> 6;
            const int64_t idx = lo + (int64_t)(threadIdx.x & 63) * step;
            const bool at_or_below = idx < hi && out_offsets[idx] <= o0;      // true for a prefix of the lanes (lane 0 always)
            const int n_below = __builtin_popcountll(__ballot(at_or_below));
            const int64_t last = lo + (int64_t)(n_below - 1) * step;
            if (last + step < hi) hi = last + step;
            lo = last;
            if (step == 1) break;
        }
        for (int64_t row = lo; row < n_rows; ++row) {
            const int64_t r0 = out_offsets[row], r1 = out_offsets[row + 1];
            if (r0 >= o1) break;
            const int64_t c0 = r0 > o0 ? r0 : o0, c1 = r1 < o1 ? r1 : o1;
            const int32_t *src = tok_tmp + in_offsets[row] - r0;       // src[o] for r0 <= o < r1
            for (int64_t o = c0 + threadIdx.x; o < c1; o += 256) {
                int32_t v = src[o];
                if (remap) v = remap[v];
                ids_out[o] = v;
                if (mask_out) mask_out[o] = 1;
            }
        }
    }
}

constexpr int kPadTile = 2048;           // cells of one row that one workgroup handles
constexpr int kPadFuseRows = 2048;       // up to this many rows every workgroup finds the longest row itself

// Longest row (lengths cut to [0, t_cap]) of the batch, by one workgroup.
__device__ __forceinline__ int32_t block_max_length(const int32_t *lengths, int64_t n_rows, int64_t t_cap,
                                                    uint32_t *red)
{
    uint32_t m = 0;
    for (int64_t i = threadIdx.x; i < n_rows; i += blockDim.x) {
        int64_t v = lengths[i];
        if (v < 0) v = 0;
        if (v > t_cap) v = t_cap;
        m = m > (uint32_t)v ? m : (uint32_t)v;
    }
    m = wave_max_u32(m);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = m;
    __syncthreads();
    uint32_t all = 0;
    for (unsigned w = 0; w < blockDim.x / 64; ++w) all = all > red[w] ? all : red[w];
    return (int32_t)all;
}

__global__ __launch_bounds__(1024) void rows_max_kernel(const int32_t *__restrict__ lengths, int64_t n_rows,
                                                        int64_t t_cap, int32_t *__restrict__ max_len)
{
    __shared__ uint32_t red[16];
    const int32_t m = block_max_length(lengths, n_rows, t_cap, red);
    if (threadIdx.x == 0) *max_len = m;
}

// Padded layout: workgroup (row, tile) writes one tile of columns of a row: the row's tokens that
// fall into it and the pad id elsewhere, up to the width.  The width is fill_to, or with
// fill_to = 0 the longest row of the batch, raised to min_width and rounded up to a multiple of
// pad_multiple (never beyond t_cap).  The longest row is found by every workgroup for itself while
// the batch is small (FUSED_MAX: the lengths are a few KB in L2, and no launch, atomic or second
// pass over the rows is needed), and read from max_len, where rows_max_kernel has put it,
// otherwise.  pad_left puts a row's tokens at the right end of the width.  OUT is the id type.
template <bool FUSED_MAX, typename OUT>
__global__ __launch_bounds__(256) void pad_rows_kernel(
    const int32_t *__restrict__ tok_tmp, const int64_t *__restrict__ in_offsets,
    const int32_t *__restrict__ lengths, int64_t n_rows, int64_t tiles_per_row,
    const int32_t *__restrict__ remap, int32_t pad_id, int64_t t_cap, int64_t fill_to, int64_t min_width,
    int64_t pad_multiple, int pad_left, OUT *__restrict__ ids, uint8_t *__restrict__ mask,
    int32_t *__restrict__ max_len, int32_t *__restrict__ width_out)
{
    __shared__ uint32_t red[4];
    int64_t width = fill_to;
    if (FUSED_MAX) {
        if (fill_to == 0 || max_len) {
            const int32_t longest = block_max_length(lengths, n_rows, t_cap, red);
            if (fill_to == 0) width = longest;
            if (max_len && blockIdx.x == 0 && threadIdx.x == 0) *max_len = longest;
        }
    } else if (fill_to == 0) {
        width = *max_len;
    }
    if (width < min_width) width = min_width;
    if (pad_multiple > 1 && width % pad_multiple) width += pad_multiple - width % pad_multiple;
    if (width > t_cap) width = t_cap;
    if (width_out && blockIdx.x == 0 && threadIdx.x == 0) *width_out = (int32_t)width;
    const int64_t n_tiles = n_rows * tiles_per_row;
    for (int64_t tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
        const int64_t row = tile / tiles_per_row;
        const int64_t c0 = (tile - row * tiles_per_row) * kPadTile;
        int64_t len = lengths[row];
        if (len < 0) len = 0;
        if (len > t_cap) len = t_cap;
        // with padding on the left a row longer than the width keeps its first `width` tokens
        const int64_t shift = pad_left ? (width > len ? width - len : 0) : 0;
        const int64_t kept = pad_left && len > width ? width : len;
        const int64_t end = pad_left ? width : (len > width ? len : width);    // cells of the row that get written
        if (c0 >= end) continue;
        const int64_t c1 = c0 + kPadTile < end ? c0 + kPadTile : end;
        const int32_t *src = tok_tmp + in_offsets[row];
        OUT *o = ids + row * t_cap;
        uint8_t *m = mask ? mask + row * t_cap : nullptr;
        for (int64_t j = c0 + threadIdx.x; j < c1; j += 256) {
            int32_t v = pad_id;
            const int64_t k = j - shift;
            const bool tok = k >= 0 && k < kept;
            if (tok) {
                v = src[k];
                if (remap) v = remap[v];
            }
            o[j] = (OUT)v;
            if (m) m[j] = tok ? 1 : 0;
        }
    }
}

static int capped_grid(int64_t want)
{
    if (want > 256 * 32) want = 256 * 32;
    return (int)(want < 1 ? 1 : want);
}

}  // namespace dnatok

using namespace dnatok;

extern "C" int dnatok_pack_ragged(const int32_t *tok_tmp, const int64_t *in_offsets,
                                  const int32_t *lengths, int64_t n_rows, const int32_t *remap,
                                  int32_t *ids_out, int64_t *out_offsets, uint8_t *mask_out,
                                  void *stream)
{
    DNATOK_REQUIRE(in_offsets && lengths && out_offsets, DNATOK_E_INVALID,
                   "dnatok_pack_ragged: null argument");
    DNATOK_REQUIRE(n_rows >= 0, DNATOK_E_INVALID, "dnatok_pack_ragged: negative row count");
    hipStream_t s = (hipStream_t)stream;
    {
        const int rc = launch_scan_lengths(lengths, n_rows, out_offsets, nullptr, 0, s);
        if (rc) return rc;
    }
    if (n_rows == 0) return DNATOK_OK;
    DNATOK_REQUIRE(tok_tmp && ids_out, DNATOK_E_INVALID, "dnatok_pack_ragged: null buffer");
    // the packed size is only known on the device: a fixed grid strides over its tiles, and
    // workgroups past the end find nothing to do
    pack_copy_kernel<<<256 * 16, 256, 0, s>>>(
        tok_tmp, in_offsets, n_rows, remap, out_offsets, ids_out, mask_out);
    DNATOK_HIP_TRY(hipGetLastError());
    return DNATOK_OK;
}

template <typename OUT>
static int launch_pad_rows(const int32_t *tok_tmp, const int64_t *in_offsets, const int32_t *lengths, int64_t n_rows,
                           const int32_t *remap, int32_t pad_id, int64_t t_cap, int64_t fill_to, int64_t min_width,
                           int64_t pad_multiple, int pad_left, OUT *ids, uint8_t *mask, int32_t *max_len,
                           int32_t *width_out, hipStream_t s)
{
    const int64_t tiles_per_row = t_cap > 0 ? (t_cap + kPadTile - 1) / kPadTile : 1;
    const int grid = capped_grid(n_rows * tiles_per_row);
    if (n_rows <= kPadFuseRows) {
        pad_rows_kernel<true, OUT><<<grid, 256, 0, s>>>(tok_tmp, in_offsets, lengths, n_rows, tiles_per_row, remap, pad_id,
                                                        t_cap, fill_to, min_width, pad_multiple, pad_left, ids, mask,
                                                        max_len, width_out);
    } else {
        if (max_len) rows_max_kernel<<<1, 1024, 0, s>>>(lengths, n_rows, t_cap, max_len);
        pad_rows_kernel<false, OUT><<<grid, 256, 0, s>>>(tok_tmp, in_offsets, lengths, n_rows, tiles_per_row, remap,
                                                         pad_id, t_cap, fill_to, min_width, pad_multiple, pad_left, ids,
                                                         mask, max_len, width_out);
    }
    DNATOK_HIP_TRY(hipGetLastError());
    return DNATOK_OK;
}

extern "C" int dnatok_pad_rows(const int32_t *tok_tmp, const int64_t *in_offsets,
                               const int32_t *lengths, int64_t n_rows, const int32_t *remap,
                               int32_t pad_id, int64_t t_cap, int64_t fill_to, int32_t *ids,
                               uint8_t *mask, int32_t *max_len, void *stream)
{
    DNATOK_REQUIRE(in_offsets && lengths && ids, DNATOK_E_INVALID, "dnatok_pad_rows: null argument");
    DNATOK_REQUIRE(n_rows >= 0 && t_cap >= 0 && fill_to >= 0 && fill_to <= t_cap, DNATOK_E_INVALID,
                   "dnatok_pad_rows: need 0 <= fill_to <= t_cap");
    DNATOK_REQUIRE(fill_to > 0 || max_len, DNATOK_E_INVALID, "dnatok_pad_rows: fill_to = 0 needs max_len");
    if (n_rows == 0) return DNATOK_OK;
    return launch_pad_rows<int32_t>(tok_tmp, in_offsets, lengths, n_rows, remap, pad_id, t_cap, fill_to, 0, 1, 0, ids,
                                    mask, max_len, nullptr, (hipStream_t)stream);
}

extern "C" int dnatok_pad_rows_as(const int32_t *tok_tmp, const int64_t *in_offsets, const int32_t *lengths,
                                  int64_t n_rows, const int32_t *remap, int32_t pad_id, int64_t t_cap,
                                  int64_t fill_to, int64_t min_width, int64_t pad_multiple, int pad_left,
                                  void *ids, int32_t id_bytes, uint8_t *mask, int32_t *max_len,
                                  int32_t *width_out, void *stream)
{
    DNATOK_REQUIRE(in_offsets && lengths && ids, DNATOK_E_INVALID, "dnatok_pad_rows_as: null argument");
    DNATOK_REQUIRE(n_rows >= 0 && t_cap >= 0 && fill_to >= 0 && fill_to <= t_cap && min_width >= 0 && min_width <= t_cap &&
                       pad_multiple >= 0,
                   DNATOK_E_INVALID, "dnatok_pad_rows_as: need 0 <= fill_to, min_width <= t_cap and pad_multiple >= 0");
    DNATOK_REQUIRE(fill_to > 0 || max_len, DNATOK_E_INVALID, "dnatok_pad_rows_as: fill_to = 0 needs max_len");
    DNATOK_REQUIRE(id_bytes == 1 || id_bytes == 2 || id_bytes == 4 || id_bytes == 8, DNATOK_E_INVALID,
                   "dnatok_pad_rows_as: id_bytes must be 1, 2, 4 or 8");
    if (n_rows == 0) return DNATOK_OK;
    hipStream_t s = (hipStream_t)stream;
#define GO(T) launch_pad_rows<T>(tok_tmp, in_offsets, lengths, n_rows, remap, pad_id, t_cap, fill_to, min_width, pad_multiple, \
                                 pad_left ? 1 : 0, (T *)ids, mask, max_len, width_out, s)
    switch (id_bytes) {
        case 1: return GO(uint8_t);
        case 2: return GO(int16_t);
        case 4: return GO(int32_t);
        default: return GO(int64_t);
    }
#undef GO
}
