// Tokenizer normalizer steps on ragged rows of bytes, on the device.
//
// The steps (strip, replace a literal, replace a run of one byte, prepend, lowercase) are grouped
// into passes of the form  [strip] [one replace] [prepend] [lowercase];  a pass is one compaction
// over the flat byte stream: every input position emits nothing, itself or the replacement,
// decided from a bounded window of its own row, every row start emits the prefix, and an
// exclusive prefix sum of the emitted sizes gives the output positions and the rows' new
// offsets.  A pass is up to four launches: count (per-lane and per-tile sizes), scan of the tile sizes (large batches),
// emit, after a small per-row launch (row table, strip bounds).  The emit kernel collects a tile's output in LDS, placed so that LDS and global addresses
// agree modulo 16, and writes it out in aligned 16-byte pieces.  Sizes after a pass are known
// only on the device: grids are sized by host-side upper bounds and workgroups beyond the real
// size find nothing to do.  HBM-bound byte work, 2 bytes read and 1 written per base and pass.
#include "common.hpp"

#include <string.h>

namespace dnatok {

constexpr int kNormThreads = 256;
constexpr int kNormPerLane = 16;                                   // positions per lane
constexpr int kNormTile = kNormThreads * kNormPerLane;             // 4096 positions per workgroup
constexpr int kNormStage = 12288;                                  // bytes of LDS for a tile's output
constexpr int kScanThreads = 1024;
constexpr int kNormSumInEmit = 8192;                              // up to this many tiles the emit kernel sums the sizes itself
constexpr int kNormSpanShift = 10;                                 // one table entry per 1024 positions (a wave's span)

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

struct PassDev {
    int32_t strip_flags;          // 0: no strip in this pass; bit 0 left, bit 1 right
    int32_t mid_kind;             // 0, DNATOK_NORM_REPLACE or DNATOK_NORM_REPLACE_RUN
    int32_t run_min;
    int32_t pattern_len, content_len, prefix_len;
    int32_t map_lower;            // emitted input bytes A-Z -> a-z (content and prefix arrive lower-cased)
    // byte strings of up to 16 bytes as two little-endian words, so that a byte is a shift and
    // not an index into an array (which would put the record into scratch memory)
    uint64_t pattern[2], content[2], prefix[2];
};

__device__ __forceinline__ uint8_t byte_of(const uint64_t (&s)[2], int k)
{
    return (uint8_t)((k < 8 ? s[0] : s[1]) >> (8 * (k & 7)));
}

enum Emit : int { kNone = 0, kSelf = 1, kContent = 2 };

__device__ __forceinline__ bool is_space(uint8_t c)
{
    return c == ' ' || (c >= 0x09 && c <= 0x0D) || (c >= 0x1C && c <= 0x1F);
}

__device__ __forceinline__ uint8_t lower_if(uint8_t c, int on)
{
    return (on && c >= 'A' && c <= 'Z') ? (uint8_t)(c + 32) : c;
}

// Byte k of a lane's own 16 bytes, held in two words.
__device__ __forceinline__ uint8_t own_byte(uint64_t w_lo, uint64_t w_hi, int k)
{
    return (uint8_t)((k < 8 ? w_lo : w_hi) >> (8 * (k & 7)));
}

// The bytes a lane looks at: its own 16 from registers, anything else from memory.  (Plain values,
// not a struct: an aggregate that is indexed at run time ends up in LDS or scratch.)
#define DNATOK_WINDOW_PARAMS const uint8_t *bytes, int64_t p0, uint64_t w_lo, uint64_t w_hi
#define DNATOK_WINDOW_ARGS bytes, p0, w_lo, w_hi

__device__ __forceinline__ uint8_t byte_at(DNATOK_WINDOW_PARAMS, int64_t q)
{
    const int64_t k = q - p0;
    return (k >= 0 && k < kNormPerLane) ? own_byte(w_lo, w_hi, (int)k) : bytes[q];
}

__device__ __forceinline__ bool match_at(const PassDev &ps, DNATOK_WINDOW_PARAMS, int64_t q, int64_t hi)
{
    if (q + ps.pattern_len > hi) return false;
    for (int j = 0; j < ps.pattern_len; ++j)
        if (byte_at(DNATOK_WINDOW_ARGS, q + j) != byte_of(ps.pattern, j)) return false;
    return true;
}

// What position p (byte c, one the replace step looks at) of a row emits; [lo, hi) is the row,
// already without what a strip removed.
__device__ __forceinline__ Emit emit_of(const PassDev &ps, DNATOK_WINDOW_PARAMS, uint8_t c, int64_t p,
                                        int64_t lo, int64_t hi)
{
    if (ps.mid_kind == DNATOK_NORM_REPLACE) {
        // the pattern has no border (no proper prefix that is also a suffix), so two matches
        // never overlap and every match is replaced
        const int m = ps.pattern_len;
        if (match_at(ps, DNATOK_WINDOW_ARGS, p, hi)) return kContent;
        for (int d = 1; d < m; ++d)
            if (p - d >= lo && byte_of(ps.pattern, d) == c && match_at(ps, DNATOK_WINDOW_ARGS, p - d, hi)) return kNone;
        return kSelf;
    }
    if (ps.mid_kind == DNATOK_NORM_REPLACE_RUN) {
        // a maximal run of the byte, at least run_min long, becomes one copy of the content
        if (c != byte_of(ps.pattern, 0)) return kSelf;
        const int n = ps.run_min;
        int back = 0, fwd = 0;
        while (back < n && p - 1 - back >= lo && byte_at(DNATOK_WINDOW_ARGS, p - 1 - back) == c) ++back;
        while (fwd < n && p + 1 + fwd < hi && byte_at(DNATOK_WINDOW_ARGS, p + 1 + fwd) == c) ++fwd;
        if (back + 1 + fwd < n) return kSelf;
        return back == 0 ? kContent : kNone;
    }
    return kSelf;
}

// First index i in [a, n] with offsets[i] >= p (offsets is non-decreasing, offsets[n] >= p).
__device__ __forceinline__ int64_t first_row_at_or_after(const int64_t *offsets, int64_t a, int64_t n, int64_t p)
{
    int64_t b = n;
    while (a < b) {
        const int64_t mid = (a + b) >> 1;
        if (offsets[mid] < p) a = mid + 1; else b = mid;
    }
    return a;
}

__device__ __forceinline__ int64_t uniform_i64(int64_t v)
{
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
    const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)((uint64_t)v >> 32));
    return (int64_t)(((uint64_t)hi << 32) | lo);
}

// Bit k of the result: byte k of x equals b.
__device__ __forceinline__ uint32_t eq_mask8(uint64_t x, uint8_t b)
{
    const uint64_t y = x ^ (0x0101010101010101ull * b);
    const uint64_t low7 = 0x7F7F7F7F7F7F7F7Full;
    const uint64_t zero = ~(((y & low7) + low7) | y | low7);        // 0x80 in every byte of y that is 0
    return (uint32_t)(((zero >> 7) * 0x0102040810204080ull) >> 56);
}

// One lane's walk over its 16 positions p0 .. p0+15 (and position `total` itself, where rows that
// end the batch start).  Returns the bytes emitted.  WRITE: dst[k] receives the k-th of them, and
// every row that starts inside the span gets its new offset, out_at + bytes emitted before it.
template <bool WRITE>
__device__ __forceinline__ uint32_t walk(const PassDev &ps, const uint8_t *bytes, bool vec_ok,
                                         const int64_t *offsets, int64_t n_rows, int64_t total,
                                         const int64_t *keep, int64_t p0, const int32_t *span_nb, int64_t out_at,
                                         uint8_t *dst, int64_t *out_offsets)
{
    if (p0 > total) return 0;
    // Everything a lane waits for is a chain of dependent loads, so the chain is kept short: the
    // table gives the row boundary at or after the wave's first position, and the three offsets
    // around it (which settle nearly every lane) and the lane's own bytes are loaded together.
    // the lane's 16 bytes as two words (shifts, no array: an indexed array would live in scratch)
    uint64_t w_lo = 0, w_hi = 0;
    if (vec_ok && p0 + kNormPerLane <= total) {
        const u32x4 v = *reinterpret_cast<const u32x4 *>(bytes + p0);
        w_lo = ((uint64_t)v.y << 32) | v.x;
        w_hi = ((uint64_t)v.w << 32) | v.z;
    } else {
#pragma unroll 1
        for (int j = 0; j < kNormPerLane; ++j) {
            if (p0 + j >= total) break;
            const uint64_t b = (uint64_t)bytes[p0 + j] << (8 * (j & 7));
            if (j < 8) w_lo |= b; else w_hi |= b;
        }
    }
    const int64_t nb0 = span_nb[p0 >> kNormSpanShift];
    const int64_t o_before = nb0 > 0 ? offsets[nb0 - 1] : 0;
    const int64_t o_at = offsets[nb0];
    const int64_t o_after = nb0 < n_rows ? offsets[nb0 + 1] : -1;
    int64_t nb, next_off, row_lo;                                   // next boundary at or after p0; the row before it
    if (o_at >= p0) { nb = nb0; next_off = o_at; row_lo = o_before; }
    else if (o_after >= p0) { nb = nb0 + 1; next_off = o_after; row_lo = o_at; }
    else {
        nb = first_row_at_or_after(offsets, nb0 + 2, n_rows, p0);
        next_off = offsets[nb];
        row_lo = offsets[nb - 1];
    }
    int64_t lo = 0, hi = 0;                                         // the current row, stripped
    if (nb > 0) {
        if (ps.strip_flags) { lo = keep[2 * (nb - 1)]; hi = keep[2 * (nb - 1) + 1]; }
        else { lo = row_lo; hi = next_off; }
    }

    // no row starts in the span and all of it is kept: only the replace step can decide anything,
    // and only at bytes it looks at
    const bool inside = next_off > p0 + (kNormPerLane - 1) && lo <= p0 && p0 + kNormPerLane <= hi;
    // bit k: the replace step looks at byte k (it can only decide something there)
    uint32_t look = 0;
    if (ps.mid_kind == DNATOK_NORM_REPLACE_RUN)
        look = eq_mask8(w_lo, byte_of(ps.pattern, 0)) | (eq_mask8(w_hi, byte_of(ps.pattern, 0)) << 8);
    if (ps.mid_kind == DNATOK_NORM_REPLACE)
        for (int d = 0; d < ps.pattern_len; ++d)
            look |= eq_mask8(w_lo, byte_of(ps.pattern, d)) | (eq_mask8(w_hi, byte_of(ps.pattern, d)) << 8);
    if (inside && look == 0) {
        if (WRITE) {
#pragma unroll
            for (int j = 0; j < kNormPerLane; ++j) dst[j] = lower_if(own_byte(w_lo, w_hi, j), ps.map_lower);
        }
        return kNormPerLane;
    }

    // Segment by segment: the row starts at the current position, then the stretch up to the next
    // row boundary (or the end of the span), of which [lo, hi) is kept.
    uint32_t sum = 0;
    int j = 0;
    for (;;) {
        if (j >= kNormPerLane) break;
        const int64_t p = p0 + j;
        while (nb <= n_rows && next_off == p) {                     // row nb starts here (nb == n_rows: the end)
            if (WRITE) out_offsets[nb] = out_at + sum;
            if (nb < n_rows) {
                if (WRITE)
                    for (int k = 0; k < ps.prefix_len; ++k) dst[sum + k] = byte_of(ps.prefix, k);
                sum += ps.prefix_len;
            }
            ++nb;
            // the boundary after the table's one is already here; others are loaded
            next_off = nb > n_rows ? -1 : (nb == nb0 + 1 ? o_after : offsets[nb]);
            if (nb <= n_rows) {
                if (ps.strip_flags) { lo = keep[2 * (nb - 1)]; hi = keep[2 * (nb - 1) + 1]; }
                else { lo = p; hi = next_off; }
            }
        }
        if (p >= total) break;
        const int64_t stop = next_off < total ? next_off : total;   // > p
        const int seg_end = stop - p0 < kNormPerLane ? (int)(stop - p0) : kNormPerLane;
        int a = lo - p0 > j ? (int)(lo - p0 < kNormPerLane ? lo - p0 : kNormPerLane) : j;
        int b = hi - p0 < seg_end ? (int)(hi - p0 > 0 ? hi - p0 : 0) : seg_end;
        if (b < a) b = a;
        // stretches the replace step does not look at are copied; the bytes between them decide
        int k = a;
        while (k < b) {
            const uint32_t rest = look >> k;
            int nxt = rest ? k + __builtin_ctz(rest) : b;
            if (nxt > b) nxt = b;
            if (WRITE)
                for (int q = k; q < nxt; ++q) dst[sum + (q - k)] = lower_if(own_byte(w_lo, w_hi, q), ps.map_lower);
            sum += nxt - k;
            k = nxt;
            if (k < b) {
                const uint8_t c = own_byte(w_lo, w_hi, k);
                const Emit e = emit_of(ps, DNATOK_WINDOW_ARGS, c, p0 + k, lo, hi);
                if (e == kSelf) {
                    if (WRITE) dst[sum] = lower_if(c, ps.map_lower);
                    sum += 1;
                } else if (e == kContent) {
                    if (WRITE)
                        for (int q = 0; q < ps.content_len; ++q) dst[sum + q] = byte_of(ps.content, q);
                    sum += ps.content_len;
                }
                ++k;
            }
        }
        j = seg_end;
    }
    return sum;
}

// Exclusive prefix sum over the workgroup's lanes and the workgroup total.
__device__ __forceinline__ int64_t block_exclusive(uint32_t v, int64_t *red, int64_t *total_out)
{
    const uint32_t inc = wave_inclusive_sum_u32(v);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (lane == 63) red[wave] = inc;
    __syncthreads();
    int64_t carry = 0, all = 0;
    for (int w = 0; w < kNormThreads / 64; ++w) {
        if (w < wave) carry += red[w];
        all += red[w];
    }
    *total_out = all;
    return carry + inc - v;
}

__global__ __launch_bounds__(kNormThreads) void norm_count_kernel(
    PassDev ps, const uint8_t *__restrict__ bytes, int vec_ok, const int64_t *__restrict__ offsets,
    int64_t n_rows, const int64_t *__restrict__ keep, const int32_t *__restrict__ span_nb,
    uint32_t *__restrict__ lane_sum, int64_t *__restrict__ tile_sum)
{
    __shared__ int64_t red[kNormThreads / 64];
    const int64_t total = offsets[n_rows];
    const int64_t tile_p0 = (int64_t)blockIdx.x * kNormTile;
    const int64_t p0 = tile_p0 + (int64_t)threadIdx.x * kNormPerLane;
    const uint32_t mine = walk<false>(ps, bytes, vec_ok != 0, offsets, n_rows, total, keep, p0, span_nb, 0, nullptr, nullptr);
    lane_sum[(int64_t)blockIdx.x * kNormThreads + threadIdx.x] = mine;
    int64_t all;
    (void)block_exclusive(mine, red, &all);
    if (threadIdx.x == 0) tile_sum[blockIdx.x] = all;
}

// tile_sum -> exclusive prefix, in place; one workgroup.
__global__ __launch_bounds__(kScanThreads) void norm_scan_kernel(int64_t *__restrict__ tile_sum, int64_t n_tiles)
{
    __shared__ int64_t part[kScanThreads / 64];
    __shared__ int64_t carry_s;
    if (threadIdx.x == 0) carry_s = 0;
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int64_t base = 0; base < n_tiles; base += kScanThreads) {
        const int64_t i = base + threadIdx.x;
        const int64_t v = i < n_tiles ? tile_sum[i] : 0;
        // inclusive scan inside the wave (a tile emits far less than 2^32 bytes, the sum of 64 may not)
        int64_t inc = v;
        for (int d = 1; d < 64; d <<= 1) {
            const int64_t up = __shfl_up(inc, d, 64);
            if (lane >= d) inc += up;
        }
        if (lane == 63) part[wave] = inc;
        __syncthreads();
        int64_t before = carry_s, all = 0;
        for (int w = 0; w < kScanThreads / 64; ++w) {
            if (w < wave) before += part[w];
            all += part[w];
        }
        if (i < n_tiles) tile_sum[i] = before + inc - v;
        __syncthreads();
        if (threadIdx.x == 0) carry_s += all;
        __syncthreads();
    }
}

__global__ __launch_bounds__(kNormThreads) void norm_emit_kernel(
    PassDev ps, const uint8_t *__restrict__ bytes, int vec_ok, const int64_t *__restrict__ offsets,
    int64_t n_rows, const int64_t *__restrict__ keep, const int32_t *__restrict__ span_nb,
    const uint32_t *__restrict__ lane_sum, const int64_t *__restrict__ tile_base, int scanned,
    uint8_t *__restrict__ out, int out_vec_ok, int64_t *__restrict__ out_offsets)
{
    __shared__ int64_t red[kNormThreads / 64];
    __shared__ __align__(16) uint8_t stage[kNormStage];
    const int64_t total = offsets[n_rows];
    const int64_t tile_p0 = (int64_t)blockIdx.x * kNormTile;
    if (tile_p0 > total) return;                                    // whole workgroup, before any barrier
    const int64_t p0 = tile_p0 + (int64_t)threadIdx.x * kNormPerLane;
    const uint32_t mine = lane_sum[(int64_t)blockIdx.x * kNormThreads + threadIdx.x];
    int64_t all;
    const int64_t before = block_exclusive(mine, red, &all);
    // the tile's output is out[g0, g0 + all): tile_base holds the scanned sizes, or, for batches of
    // few tiles, the sizes themselves, summed here (one launch less)
    int64_t g0;
    if (scanned) {
        g0 = tile_base[blockIdx.x];
    } else {
        int64_t part = 0;
        for (int64_t t = threadIdx.x; t < (int64_t)blockIdx.x; t += kNormThreads) part += tile_base[t];
        for (int d = 32; d; d >>= 1) part += __shfl_xor(part, d, 64);
        __syncthreads();                                            // red is read by block_exclusive above
        if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = part;
        __syncthreads();
        g0 = red[0] + red[1] + red[2] + red[3];
    }
    const int shift = (int)(g0 & 15);
    const bool staged = out_vec_ok && all + 16 <= kNormStage;       // same for every lane
    if (!staged) {
        (void)walk<true>(ps, bytes, vec_ok != 0, offsets, n_rows, total, keep, p0, span_nb, g0 + before,
                         out + g0 + before, out_offsets);
        return;
    }
    (void)walk<true>(ps, bytes, vec_ok != 0, offsets, n_rows, total, keep, p0, span_nb, g0 + before,
                     stage + shift + before, out_offsets);
    __syncthreads();
    // stage[k] belongs at out[(g0 & ~15) + k]: aligned 16-byte pieces inside [g0, g1), bytes at the rims
    const int64_t g1 = g0 + all;
    const int64_t first = g0 & ~(int64_t)15;
    const int n_pieces = (int)((g1 - first + 15) >> 4);
    for (int k = threadIdx.x; k < n_pieces; k += kNormThreads) {
        const int64_t at = first + (int64_t)k * 16;
        if (at >= g0 && at + 16 <= g1) {
            *reinterpret_cast<u32x4 *>(out + at) = *reinterpret_cast<const u32x4 *>(stage + k * 16);
        } else {
            for (int j = 0; j < 16; ++j)
                if (at + j >= g0 && at + j < g1) out[at + j] = stage[k * 16 + j];
        }
    }
}

// Per row boundary i (i = n_rows is the end of the batch): span_nb[s] = i for every span of 1024
// positions whose first position lies in (offsets[i-1], offsets[i]], so that span_nb[s] is the first
// boundary at or after the span's start.  With a strip step also [keep_lo, keep_hi) of row i, the
// row without leading / trailing whitespace.
__global__ __launch_bounds__(kNormThreads) void norm_rows_kernel(
    const uint8_t *__restrict__ bytes, const int64_t *__restrict__ offsets, int64_t n_rows, int flags,
    int32_t *__restrict__ span_nb, int64_t *__restrict__ keep)
{
    const int64_t i = (int64_t)blockIdx.x * kNormThreads + threadIdx.x;
    if (i > n_rows) return;
    const int64_t at = offsets[i];
    const int64_t first = i > 0 ? (offsets[i - 1] >> kNormSpanShift) + 1 : 0;
    for (int64_t sp = first; sp <= (at >> kNormSpanShift); ++sp) span_nb[sp] = (int32_t)i;
    if (flags == 0 || i == n_rows) return;
    int64_t lo = at, hi = offsets[i + 1];
    if (flags & 1) while (lo < hi && is_space(bytes[lo])) ++lo;
    if (flags & 2) while (hi > lo && is_space(bytes[hi - 1])) --hi;
    keep[2 * i] = lo;
    keep[2 * i + 1] = hi;
}

__global__ __launch_bounds__(kNormThreads) void norm_copy_kernel(
    const uint8_t *__restrict__ bytes, const int64_t *__restrict__ offsets, int64_t n_rows, int64_t bound,
    uint8_t *__restrict__ out, int64_t *__restrict__ out_offsets)
{
    const int64_t total = offsets[n_rows];
    for (int64_t i = (int64_t)blockIdx.x * kNormThreads + threadIdx.x; i < bound; i += (int64_t)gridDim.x * kNormThreads) {
        if (i < total) out[i] = bytes[i];
        if (i <= n_rows) out_offsets[i] = offsets[i];
    }
}

static bool has_border(const uint8_t *p, int m)
{
    for (int k = 1; k < m; ++k)
        if (memcmp(p, p + m - k, (size_t)k) == 0) return true;
    return false;
}

static int check_step(const dnatok_norm_step &s, int i)
{
    DNATOK_REQUIRE(s.pattern_len >= 0 && s.pattern_len <= DNATOK_NORM_MAX_BYTES && s.content_len >= 0 &&
                       s.content_len <= DNATOK_NORM_MAX_BYTES,
                   DNATOK_E_INVALID, "normalizer step %d: pattern / content longer than %d bytes", i,
                   DNATOK_NORM_MAX_BYTES);
    switch (s.kind) {
    case DNATOK_NORM_STRIP:
    case DNATOK_NORM_PREPEND:
    case DNATOK_NORM_LOWERCASE:
        return DNATOK_OK;
    case DNATOK_NORM_REPLACE:
        DNATOK_REQUIRE(s.pattern_len >= 1, DNATOK_E_INVALID, "normalizer step %d: empty pattern", i);
        DNATOK_REQUIRE(!has_border(s.pattern, s.pattern_len), DNATOK_E_INVALID,
                       "normalizer step %d: the pattern overlaps itself (a prefix equals a suffix); "
                       "such a replace is sequential and is not done on the device", i);
        return DNATOK_OK;
    case DNATOK_NORM_REPLACE_RUN:
        DNATOK_REQUIRE(s.pattern_len == 1 && s.flags >= 1 && s.flags <= 64, DNATOK_E_INVALID,
                       "normalizer step %d: a run step takes one byte and a minimum length of 1..64", i);
        return DNATOK_OK;
    default:
        dnatok::set_error("normalizer step %d: unknown kind %d", i, (int)s.kind);
        return DNATOK_E_INVALID;
    }
}

// Upper bounds of the total and of the longest row after a step.
static void grow(const dnatok_norm_step &s, int64_t n_rows, int64_t &total, int64_t &max_len)
{
    auto repl = [](int64_t n, int64_t unit, int64_t content) {
        return content > unit ? (n / unit) * content + n % unit : n;
    };
    if (s.kind == DNATOK_NORM_PREPEND) { total += n_rows * s.content_len; max_len += s.content_len; }
    if (s.kind == DNATOK_NORM_REPLACE) { total = repl(total, s.pattern_len, s.content_len); max_len = repl(max_len, s.pattern_len, s.content_len); }
    if (s.kind == DNATOK_NORM_REPLACE_RUN) { total = repl(total, s.flags, s.content_len); max_len = repl(max_len, s.flags, s.content_len); }
}

// Position of a step inside a pass: strip, then one replace, then prepend, then lowercase.
static int level_of(int kind)
{
    switch (kind) {
    case DNATOK_NORM_STRIP: return 1;
    case DNATOK_NORM_REPLACE:
    case DNATOK_NORM_REPLACE_RUN: return 2;
    case DNATOK_NORM_PREPEND: return 3;
    default: return 4;
    }
}

struct HostPass {
    PassDev dev;
    int64_t bound_in;               // upper bound of the bytes the pass reads
};

// Groups the steps into passes; returns their number (at most n_steps).
static int make_passes(const dnatok_norm_step *steps, int n_steps, int64_t n_rows, int64_t total,
                       int64_t max_len, HostPass *passes, int64_t *out_total, int64_t *out_max_len, int64_t *cap)
{
    int n = 0, level = 0;
    int64_t t = total, m = max_len, c = total;
    for (int i = 0; i < n_steps; ++i) {
        const dnatok_norm_step &s = steps[i];
        if (s.kind == DNATOK_NORM_STRIP && (s.flags & 3) == 0) continue;
        const int lv = level_of(s.kind);
        if (n == 0 || lv <= level) {
            if (passes) { memset(&passes[n], 0, sizeof(HostPass)); passes[n].bound_in = t; }
            ++n;
        }
        level = lv;
        if (passes) {
            PassDev &d = passes[n - 1].dev;
            if (s.kind == DNATOK_NORM_STRIP) d.strip_flags = s.flags & 3;
            if (s.kind == DNATOK_NORM_REPLACE || s.kind == DNATOK_NORM_REPLACE_RUN) {
                d.mid_kind = s.kind;
                d.run_min = s.flags;
                d.pattern_len = s.pattern_len;
                d.content_len = s.content_len;
                memcpy(d.pattern, s.pattern, sizeof(d.pattern));      // little-endian host: byte k is bits 8k.. of the words
                memcpy(d.content, s.content, sizeof(d.content));
            }
            if (s.kind == DNATOK_NORM_PREPEND) { d.prefix_len = s.content_len; memcpy(d.prefix, s.content, sizeof(d.prefix)); }
            if (s.kind == DNATOK_NORM_LOWERCASE) {
                d.map_lower = 1;
                uint8_t *cb = reinterpret_cast<uint8_t *>(d.content), *pb = reinterpret_cast<uint8_t *>(d.prefix);
                for (int k = 0; k < DNATOK_NORM_MAX_BYTES; ++k) {
                    if (cb[k] >= 'A' && cb[k] <= 'Z') cb[k] += 32;
                    if (pb[k] >= 'A' && pb[k] <= 'Z') pb[k] += 32;
                }
            }
        }
        grow(s, n_rows, t, m);
        if (t > c) c = t;
    }
    if (out_total) *out_total = t;
    if (out_max_len) *out_max_len = m;
    if (cap) *cap = c;
    return n;
}

struct NormPlan {
    int64_t cap;                     // bytes of each intermediate buffer
    int64_t out_total, out_max_len;
    int64_t n_tiles;                 // tiles of the largest pass
    size_t off_a, off_b, off_offs_a, off_offs_b, off_tiles, off_lanes, off_spans, off_keep, bytes;
};

static NormPlan plan_for(const dnatok_norm_step *steps, int n_steps, int64_t n_rows, int64_t total, int64_t max_len)
{
    NormPlan p{};
    (void)make_passes(steps, n_steps, n_rows, total, max_len, nullptr, &p.out_total, &p.out_max_len, &p.cap);
    p.n_tiles = p.cap / kNormTile + 1;
    auto up = [](size_t v) { return (v + 255) & ~(size_t)255; };
    size_t at = 0;
    p.off_a = at; at = up(at + (size_t)p.cap);
    p.off_b = at; at = up(at + (size_t)p.cap);
    p.off_offs_a = at; at = up(at + sizeof(int64_t) * (size_t)(n_rows + 1));
    p.off_offs_b = at; at = up(at + sizeof(int64_t) * (size_t)(n_rows + 1));
    p.off_tiles = at; at = up(at + sizeof(int64_t) * (size_t)p.n_tiles);
    p.off_lanes = at; at = up(at + sizeof(uint32_t) * (size_t)p.n_tiles * kNormThreads);
    p.off_spans = at; at = up(at + sizeof(int32_t) * (size_t)((p.cap >> kNormSpanShift) + 2));
    p.off_keep = at; at = up(at + sizeof(int64_t) * 2 * (size_t)(n_rows > 0 ? n_rows : 1));
    p.bytes = at;
    return p;
}

}  // namespace dnatok

using namespace dnatok;

extern "C" int dnatok_normalize_bounds(const dnatok_norm_step *steps_h, int32_t n_steps, int64_t n_rows,
                                       int64_t total, int64_t max_len, int64_t *out_total,
                                       int64_t *out_max_len, size_t *scratch_bytes)
{
    DNATOK_REQUIRE(n_steps >= 0 && (steps_h || n_steps == 0) && n_rows >= 0 && total >= 0 && max_len >= 0,
                   DNATOK_E_INVALID, "dnatok_normalize_bounds: bad argument");
    for (int i = 0; i < n_steps; ++i) {
        const int rc = check_step(steps_h[i], i);
        if (rc != DNATOK_OK) return rc;
    }
    const NormPlan p = plan_for(steps_h, n_steps, n_rows, total, max_len);
    if (out_total) *out_total = p.out_total;
    if (out_max_len) *out_max_len = p.out_max_len;
    if (scratch_bytes) *scratch_bytes = p.bytes;
    return DNATOK_OK;
}

extern "C" int dnatok_normalize_rows(const dnatok_norm_step *steps_h, int32_t n_steps, const uint8_t *bytes,
                                     const int64_t *offsets, int64_t n_rows, int64_t total, int64_t max_len,
                                     uint8_t *out_bytes, int64_t out_capacity, int64_t *out_offsets,
                                     void *scratch, size_t scratch_bytes, void *stream)
{
    DNATOK_REQUIRE(n_steps >= 0 && n_steps <= 64 && (steps_h || n_steps == 0) && n_rows >= 0 && total >= 0 &&
                       max_len >= 0,
                   DNATOK_E_INVALID, "dnatok_normalize_rows: bad argument (at most 64 steps)");
    DNATOK_REQUIRE(offsets && out_offsets, DNATOK_E_INVALID, "dnatok_normalize_rows: null offsets");
    for (int i = 0; i < n_steps; ++i) {
        const int rc = check_step(steps_h[i], i);
        if (rc != DNATOK_OK) return rc;
    }
    const NormPlan p = plan_for(steps_h, n_steps, n_rows, total, max_len);
    DNATOK_REQUIRE(out_capacity >= p.out_total, DNATOK_E_SCRATCH,
                   "dnatok_normalize_rows: output holds %lld bytes, up to %lld needed", (long long)out_capacity,
                   (long long)p.out_total);
    DNATOK_REQUIRE((bytes || total == 0) && (out_bytes || p.out_total == 0), DNATOK_E_INVALID,
                   "dnatok_normalize_rows: null buffer");
    HostPass passes[64];
    const int n_passes = make_passes(steps_h, n_steps, n_rows, total, max_len, passes, nullptr, nullptr, nullptr);
    DNATOK_REQUIRE(n_passes == 0 || (scratch && scratch_bytes >= p.bytes), DNATOK_E_SCRATCH,
                   "dnatok_normalize_rows: scratch holds %zu bytes, %zu needed", scratch_bytes, p.bytes);
    DNATOK_REQUIRE(p.n_tiles < (int64_t)1 << 31 && n_rows < ((int64_t)1 << 31) - 1, DNATOK_E_TOO_LARGE,
                   "dnatok_normalize_rows: input too large");
    hipStream_t s = (hipStream_t)stream;
    uint8_t *base = (uint8_t *)scratch;

    if (n_passes == 0) {
        const int64_t bound = (total > n_rows + 1 ? total : n_rows + 1);
        const int64_t want = (bound + kNormThreads - 1) / kNormThreads;
        norm_copy_kernel<<<(int)(want < 8192 ? want : 8192), kNormThreads, 0, s>>>(bytes, offsets, n_rows, bound,
                                                                                 out_bytes, out_offsets);
        DNATOK_HIP_TRY(hipGetLastError());
        return DNATOK_OK;
    }

    const uint8_t *cur = bytes;
    const int64_t *cur_off = offsets;
    int64_t *tiles = (int64_t *)(base + p.off_tiles);
    uint32_t *lanes = (uint32_t *)(base + p.off_lanes);
    int64_t *keep = (int64_t *)(base + p.off_keep);
    int32_t *spans = (int32_t *)(base + p.off_spans);
    for (int i = 0; i < n_passes; ++i) {
        const PassDev &ps = passes[i].dev;
        const bool last = i == n_passes - 1;
        uint8_t *dst = last ? out_bytes : base + ((i & 1) ? p.off_b : p.off_a);
        int64_t *dst_off = last ? out_offsets : (int64_t *)(base + ((i & 1) ? p.off_offs_b : p.off_offs_a));
        norm_rows_kernel<<<(int)(n_rows / kNormThreads + 1), kNormThreads, 0, s>>>(cur, cur_off, n_rows, ps.strip_flags,
                                                                                 spans, keep);
        const int64_t n_tiles = passes[i].bound_in / kNormTile + 1;   // covers position `total` itself
        const int vec_in = ((uintptr_t)cur & 15) == 0, vec_out = ((uintptr_t)dst & 15) == 0;
        norm_count_kernel<<<(int)n_tiles, kNormThreads, 0, s>>>(ps, cur, vec_in, cur_off, n_rows, keep, spans, lanes, tiles);
        const int scanned = n_tiles > kNormSumInEmit;
        if (scanned) norm_scan_kernel<<<1, kScanThreads, 0, s>>>(tiles, n_tiles);
        norm_emit_kernel<<<(int)n_tiles, kNormThreads, 0, s>>>(ps, cur, vec_in, cur_off, n_rows, keep, spans, lanes, tiles,
                                                               scanned, dst, vec_out, dst_off);
        DNATOK_HIP_TRY(hipGetLastError());
        cur = dst;
        cur_off = dst_off;
    }
    return DNATOK_OK;
}
