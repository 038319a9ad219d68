// Tokenizer normalizer steps on ragged rows of bytes, on the device.
//
// Each step (strip, replace a literal, replace a run of one byte, prepend, byte map) is one
// compaction pass over the flat byte stream: every input position emits nothing, itself or the
// step's replacement bytes, decided from a bounded window of its own row; an exclusive prefix
// sum of the emitted sizes gives the output position, and the rows' new offsets fall out of the
// same walk.  A pass is three launches (count per tile, scan of the tile sums, emit); the sizes
// after a step are known only on the device, so grids are sized by host-side upper bounds and
// workgroups beyond the real size find nothing to do.  HBM-bound byte work: about 2 bytes read
// and 1 written per base and pass, small beside the merge engine that follows.
#include "common.hpp"

#include <string.h>

namespace dnatok {

constexpr int kNormThreads = 256;
constexpr int kNormPerLane = 16;                                   // positions per lane
constexpr int kNormTile = kNormThreads * kNormPerLane;             // 4096 positions per workgroup
constexpr int kScanThreads = 1024;

struct StepDev {
    int32_t kind, flags, pattern_len, content_len;
    uint8_t pattern[DNATOK_NORM_MAX_BYTES];
    uint8_t content[DNATOK_NORM_MAX_BYTES];
    uint8_t map_lower;                                              // emitted bytes A-Z -> a-z
};

enum Emit : int { kNone = 0, kSelf = 1, kContent = 2 };

__device__ __forceinline__ bool is_space(uint8_t c)
{
    return c == ' ' || (c >= 0x09 && c <= 0x0D) || (c >= 0x1C && c <= 0x1F);
}

__device__ __forceinline__ bool match_at(const StepDev &st, const uint8_t *bytes, int64_t q, int64_t hi)
{
    if (q + st.pattern_len > hi) return false;
    for (int j = 0; j < st.pattern_len; ++j)
        if (bytes[q + j] != st.pattern[j]) return false;
    return true;
}

// What position p of the row [lo, hi) emits.  [keep_lo, keep_hi) is the row without the
// whitespace a strip step removes.
__device__ __forceinline__ Emit emit_of(const StepDev &st, const uint8_t *bytes, uint8_t c, int64_t p,
                                        int64_t lo, int64_t hi, int64_t keep_lo, int64_t keep_hi)
{
    switch (st.kind) {
    case DNATOK_NORM_STRIP:
        return (p >= keep_lo && p < keep_hi) ? kSelf : kNone;
    case DNATOK_NORM_REPLACE: {
        // the pattern has no border (no proper prefix that is also a suffix), so two matches
        // never overlap and every match is replaced
        const int m = st.pattern_len;
        bool maybe = false;
        for (int d = 0; d < m; ++d) maybe |= st.pattern[d] == c;
        if (!maybe) return kSelf;
        if (match_at(st, bytes, p, hi)) return kContent;
        for (int d = 1; d < m; ++d)
            if (p - d >= lo && st.pattern[d] == c && match_at(st, bytes, p - d, hi)) return kNone;
        return kSelf;
    }
    case DNATOK_NORM_REPLACE_RUN: {
        // a maximal run of the byte, at least `flags` long, becomes one copy of the content
        if (c != st.pattern[0]) return kSelf;
        const int n = st.flags;
        int back = 0, fwd = 0;
        while (back < n && p - 1 - back >= lo && bytes[p - 1 - back] == c) ++back;
        while (fwd < n && p + 1 + fwd < hi && bytes[p + 1 + fwd] == c) ++fwd;
        if (back + 1 + fwd < n) return kSelf;
        return back == 0 ? kContent : kNone;
    }
    default:                                                        // prepend, byte map
        return kSelf;
    }
}

// First index i in [0, n] with offsets[i] >= p (offsets is non-decreasing, offsets[n] >= p).
__device__ __forceinline__ int64_t first_row_at_or_after(const int64_t *offsets, int64_t n, int64_t p)
{
    int64_t a = 0, b = n;
    while (a < b) {
        const int64_t mid = (a + b) >> 1;
        if (offsets[mid] < p) a = mid + 1; else b = mid;
    }
    return a;
}

// One lane's walk over its 16 positions.  WRITE = false: returns the bytes they emit.
// WRITE = true: emits them from output position `at` on and writes the new offset (and the
// prefix) of every row that starts inside the lane's span.
template <bool WRITE>
__device__ __forceinline__ int64_t walk(const StepDev &st, const uint8_t *bytes, const int64_t *offsets,
                                        int64_t n_rows, int64_t total, const int64_t *keep, int64_t p0,
                                        int64_t at, uint8_t *out, int64_t *out_offsets)
{
    if (p0 > total) return 0;
    const int plen = st.kind == DNATOK_NORM_PREPEND ? st.content_len : 0;
    int64_t nb = first_row_at_or_after(offsets, n_rows, p0);        // next row boundary at or after p0
    int64_t next_off = offsets[nb];
    int64_t lo = nb > 0 ? offsets[nb - 1] : 0;
    int64_t keep_lo = 0, keep_hi = 0;
    if (st.kind == DNATOK_NORM_STRIP && nb > 0) { keep_lo = keep[2 * (nb - 1)]; keep_hi = keep[2 * (nb - 1) + 1]; }
    int64_t sum = 0;
    for (int j = 0; j < kNormPerLane; ++j) {
        const int64_t p = p0 + j;
        if (p > total) break;
        while (nb <= n_rows && next_off == p) {                     // row nb starts here (nb == n_rows: the end)
            if (WRITE) {
                const int64_t row_at = at + sum + nb * plen;
                out_offsets[nb] = row_at;
                if (nb < n_rows)
                    for (int k = 0; k < plen; ++k) out[row_at + k] = st.content[k];
            }
            lo = p;
            if (st.kind == DNATOK_NORM_STRIP && nb < n_rows) { keep_lo = keep[2 * nb]; keep_hi = keep[2 * nb + 1]; }
            ++nb;
            next_off = nb <= n_rows ? offsets[nb] : -1;
        }
        if (p == total) break;
        const uint8_t c = bytes[p];
        const Emit e = emit_of(st, bytes, c, p, lo, next_off, keep_lo, keep_hi);
        if (e == kSelf) {
            if (WRITE) out[at + sum + nb * plen] = (st.map_lower && c >= 'A' && c <= 'Z') ? (uint8_t)(c + 32) : c;
            sum += 1;
        } else if (e == kContent) {
            if (WRITE)
                for (int k = 0; k < st.content_len; ++k) out[at + sum + nb * plen + k] = st.content[k];
            sum += st.content_len;
        }
    }
    return sum;
}

// Exclusive prefix sum over the workgroup's lanes (in place) and the workgroup total.
__device__ __forceinline__ int64_t block_exclusive(int64_t v, int64_t *red, int64_t *total_out)
{
    // emitted sizes per lane fit 32 bits (16 positions x at most 16 bytes)
    const uint32_t inc = wave_inclusive_sum_u32((uint32_t)v);
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
    StepDev st, const uint8_t *__restrict__ bytes, const int64_t *__restrict__ offsets, int64_t n_rows,
    const int64_t *__restrict__ keep, int64_t *__restrict__ tile_sum)
{
    __shared__ int64_t red[kNormThreads / 64];
    const int64_t total = offsets[n_rows];
    const int64_t p0 = (int64_t)blockIdx.x * kNormTile + (int64_t)threadIdx.x * kNormPerLane;
    const int64_t mine = walk<false>(st, bytes, offsets, n_rows, total, keep, p0, 0, nullptr, nullptr);
    int64_t all;
    (void)block_exclusive(mine, red, &all);
    if (threadIdx.x == 0) tile_sum[blockIdx.x] = all;
}

// tile_sum -> exclusive prefix, in place; one workgroup.
__global__ __launch_bounds__(kScanThreads) void norm_scan_kernel(int64_t *__restrict__ tile_sum, int64_t n_tiles)
{
    __shared__ int64_t part[kScanThreads];
    __shared__ int64_t carry_s;
    if (threadIdx.x == 0) carry_s = 0;
    __syncthreads();
    for (int64_t base = 0; base < n_tiles; base += kScanThreads) {
        const int64_t i = base + threadIdx.x;
        const int64_t v = i < n_tiles ? tile_sum[i] : 0;
        part[threadIdx.x] = v;
        __syncthreads();
        for (int d = 1; d < kScanThreads; d <<= 1) {                // Hillis-Steele, inclusive
            const int64_t add = threadIdx.x >= (unsigned)d ? part[threadIdx.x - d] : 0;
            __syncthreads();
            part[threadIdx.x] += add;
            __syncthreads();
        }
        const int64_t carry = carry_s;
        if (i < n_tiles) tile_sum[i] = carry + part[threadIdx.x] - v;
        __syncthreads();
        if (threadIdx.x == kScanThreads - 1) carry_s = carry + part[threadIdx.x];
        __syncthreads();
    }
}

__global__ __launch_bounds__(kNormThreads) void norm_emit_kernel(
    StepDev st, const uint8_t *__restrict__ bytes, const int64_t *__restrict__ offsets, int64_t n_rows,
    const int64_t *__restrict__ keep, const int64_t *__restrict__ tile_base,
    uint8_t *__restrict__ out, int64_t *__restrict__ out_offsets)
{
    __shared__ int64_t red[kNormThreads / 64];
    const int64_t total = offsets[n_rows];
    const int64_t p0 = (int64_t)blockIdx.x * kNormTile + (int64_t)threadIdx.x * kNormPerLane;
    const int64_t mine = walk<false>(st, bytes, offsets, n_rows, total, keep, p0, 0, nullptr, nullptr);
    int64_t all;
    const int64_t before = block_exclusive(mine, red, &all);
    (void)walk<true>(st, bytes, offsets, n_rows, total, keep, p0, tile_base[blockIdx.x] + before, out, out_offsets);
}

// Per row: [keep_lo, keep_hi) = the row without leading / trailing whitespace.
__global__ __launch_bounds__(kNormThreads) void norm_strip_bounds_kernel(
    const uint8_t *__restrict__ bytes, const int64_t *__restrict__ offsets, int64_t n_rows, int flags,
    int64_t *__restrict__ keep)
{
    const int64_t b = (int64_t)blockIdx.x * kNormThreads + threadIdx.x;
    if (b >= n_rows) return;
    int64_t lo = offsets[b], hi = offsets[b + 1];
    if (flags & 1) while (lo < hi && is_space(bytes[lo])) ++lo;
    if (flags & 2) while (hi > lo && is_space(bytes[hi - 1])) --hi;
    keep[2 * b] = lo;
    keep[2 * b + 1] = hi;
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

struct NormPlan {
    int64_t cap;                     // bytes of each intermediate buffer
    int64_t out_total, out_max_len;
    int64_t n_tiles;                 // tiles of the largest pass
    size_t off_a, off_b, off_offs_a, off_offs_b, off_tiles, off_keep, bytes;
};

static NormPlan plan_for(const dnatok_norm_step *steps, int n_steps, int64_t n_rows, int64_t total, int64_t max_len)
{
    NormPlan p{};
    int64_t t = total, m = max_len, cap = total;
    for (int i = 0; i < n_steps; ++i) {
        grow(steps[i], n_rows, t, m);
        if (t > cap) cap = t;
    }
    p.cap = cap;
    p.out_total = t;
    p.out_max_len = m;
    p.n_tiles = cap / kNormTile + 1;
    auto up = [](size_t v) { return (v + 255) & ~(size_t)255; };
    size_t at = 0;
    p.off_a = at; at = up(at + (size_t)cap);
    p.off_b = at; at = up(at + (size_t)cap);
    p.off_offs_a = at; at = up(at + sizeof(int64_t) * (size_t)(n_rows + 1));
    p.off_offs_b = at; at = up(at + sizeof(int64_t) * (size_t)(n_rows + 1));
    p.off_tiles = at; at = up(at + sizeof(int64_t) * (size_t)p.n_tiles);
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
    DNATOK_REQUIRE(n_steps >= 0 && (steps_h || n_steps == 0) && n_rows >= 0 && total >= 0 && max_len >= 0,
                   DNATOK_E_INVALID, "dnatok_normalize_rows: bad argument");
    DNATOK_REQUIRE(offsets && out_offsets, DNATOK_E_INVALID, "dnatok_normalize_rows: null offsets");
    for (int i = 0; i < n_steps; ++i) {
        const int rc = check_step(steps_h[i], i);
        if (rc != DNATOK_OK) return rc;
    }
    const NormPlan p = plan_for(steps_h, n_steps, n_rows, total, max_len);
    DNATOK_REQUIRE(out_capacity >= p.out_total, DNATOK_E_SCRATCH,
                   "dnatok_normalize_rows: output holds %lld bytes, up to %lld needed", (long long)out_capacity,
                   (long long)p.out_total);
    DNATOK_REQUIRE(p.out_total == 0 || (bytes && out_bytes) || total == 0, DNATOK_E_INVALID,
                   "dnatok_normalize_rows: null buffer");
    DNATOK_REQUIRE(n_steps == 0 || (scratch && scratch_bytes >= p.bytes), DNATOK_E_SCRATCH,
                   "dnatok_normalize_rows: scratch holds %zu bytes, %zu needed", scratch_bytes, p.bytes);
    hipStream_t s = (hipStream_t)stream;
    uint8_t *base = (uint8_t *)scratch;

    if (n_steps == 0) {
        const int64_t bound = (total > n_rows + 1 ? total : n_rows + 1);
        const int grid = (int)((bound + kNormThreads - 1) / kNormThreads < 8192 ? (bound + kNormThreads - 1) / kNormThreads : 8192);
        norm_copy_kernel<<<grid, kNormThreads, 0, s>>>(bytes, offsets, n_rows, bound, out_bytes, out_offsets);
        DNATOK_HIP_TRY(hipGetLastError());
        return DNATOK_OK;
    }

    const uint8_t *cur = bytes;
    const int64_t *cur_off = offsets;
    int64_t bound_total = total, bound_max = max_len;
    int64_t *tiles = (int64_t *)(base + p.off_tiles);
    int64_t *keep = (int64_t *)(base + p.off_keep);
    for (int i = 0; i < n_steps; ++i) {
        const dnatok_norm_step &h = steps_h[i];
        StepDev st{};
        st.kind = h.kind;
        st.flags = h.flags;
        st.pattern_len = h.pattern_len;
        st.content_len = h.content_len;
        memcpy(st.pattern, h.pattern, sizeof(st.pattern));
        memcpy(st.content, h.content, sizeof(st.content));
        st.map_lower = h.kind == DNATOK_NORM_LOWERCASE;
        const bool last = i == n_steps - 1;
        uint8_t *dst = last ? out_bytes : base + ((i & 1) ? p.off_b : p.off_a);
        int64_t *dst_off = last ? out_offsets : (int64_t *)(base + ((i & 1) ? p.off_offs_b : p.off_offs_a));
        if (h.kind == DNATOK_NORM_STRIP && n_rows > 0) {
            norm_strip_bounds_kernel<<<(int)((n_rows + kNormThreads - 1) / kNormThreads), kNormThreads, 0, s>>>(
                cur, cur_off, n_rows, h.flags, keep);
        }
        const int64_t n_tiles = bound_total / kNormTile + 1;       // covers position `total` itself
        DNATOK_REQUIRE(n_tiles < (int64_t)1 << 31, DNATOK_E_TOO_LARGE, "dnatok_normalize_rows: input too large");
        norm_count_kernel<<<(int)n_tiles, kNormThreads, 0, s>>>(st, cur, cur_off, n_rows, keep, tiles);
        norm_scan_kernel<<<1, kScanThreads, 0, s>>>(tiles, n_tiles);
        norm_emit_kernel<<<(int)n_tiles, kNormThreads, 0, s>>>(st, cur, cur_off, n_rows, keep, tiles, dst, dst_off);
        DNATOK_HIP_TRY(hipGetLastError());
        grow(h, n_rows, bound_total, bound_max);
        cur = dst;
        cur_off = dst_off;
    }
    return DNATOK_OK;
}
