// Non-overlapping k-mer encoder with per-window fallback, tail handling, padding and mask.
//
// Persistent workgroups stage the tables in LDS once; after that every wave works alone:
// it takes a row and walks it in steps of 256 units (a unit is a k-base window, or one of
// the trailing len % k characters).  Each lane owns 4 consecutive units: it loads its 4k
// bytes, turns them into base-5 digits through the LDS digit table, and looks the window up
// in the LDS table of the 4^k N-free windows.
//
//   * Step without exceptions (the common case): every lane holds 4 plain windows, so token
//     positions are known without a scan and each lane issues one 16-byte id store and one
//     4-byte mask store (a wave covers 1 KiB + 256 B contiguous).
//   * Step with exceptions (a window holding N or a byte outside the alphabet, a window
//     without an id, the ragged end of a row): unit token counts are prefix-summed across
//     the wave with a DPP scan (no barrier) and every lane writes at its own offset.  When
//     the table spells every non-plain window character by character (the usual grid-aligned
//     tokenizer), the spelled tokens come from 5 LDS entries; otherwise from the global
//     5^k entry table and its expansion lists.
//
// Traffic: 1 byte read per base, 5 bytes written per token.
#include "common.hpp"

#include <limits.h>
#include <string.h>
#include <vector>

struct dnatok_kmer_table {
    int k;
    int64_t pow4, pow5;
    int32_t pad_id, missing_id;
    int chars_mode;          // every non-plain window expands to its own characters
    void *blob;              // one device allocation holding all tables
    int8_t *digit;           // [256]
    int32_t *single;         // [256]
    int32_t *lut4;           // [4^k]  id of an ACGT-only window, or -1
    int2 *entry;             // [5^k]  {id, 0} | {-len, offset into flat} | {INT_MIN, 0} = nothing known
    int32_t *flat;           // expansion lists
};

namespace dnatok {

struct KmerArgs {
    const int8_t *digit;
    const int32_t *single, *lut4;
    const int2 *entry;
    const int32_t *flat;
    int32_t pad_id, missing_id;
};

constexpr int kKmerThreads = 256;
constexpr int kUnitsPerLane = 4;
constexpr int kWaveUnits = 64 * kUnitsPerLane;          // units one wave handles per step

// LDS digit entries: 0..3 for A C G T; flags above every window code (4^8 = 1 << 16) for N and
// for a byte outside the alphabet, so that "window code < 4^k" means "k plain bases".
constexpr uint32_t kDigN = 1u << 16;
constexpr uint32_t kDigBad = 1u << 17;

typedef int32_t int4v __attribute__((ext_vector_type(4)));
// the same vectors at element alignment: a row's token position is not a multiple of 4 once a
// window has expanded, and global stores only need the element alignment
typedef int32_t int4v_a4 __attribute__((ext_vector_type(4), aligned(4)));
typedef uint32_t u32_a1 __attribute__((aligned(1)));

__global__ void zero_i32_kernel(int32_t *p) { *p = 0; }

__device__ __forceinline__ void store4(int32_t *out, uint8_t *mout, int p, const int32_t *t)
{
    int4v_a4 v = {t[0], t[1], t[2], t[3]};
    __builtin_nontemporal_store(v, reinterpret_cast<int4v_a4 *>(out + p));
    if (mout) __builtin_nontemporal_store((u32_a1)0x01010101u, reinterpret_cast<u32_a1 *>(mout + p));
}

__device__ __forceinline__ void store1(int32_t *out, uint8_t *mout, int p, int t_cap, int32_t v)
{
    if (p < t_cap) {
        out[p] = v;
        if (mout) mout[p] = 1;
    }
}

typedef int32_t int2v_a4 __attribute__((ext_vector_type(2), aligned(4)));
typedef uint16_t u16_a1 __attribute__((aligned(1)));

// N consecutive tokens (a spelled window) with as few stores as possible.
template <int N>
__device__ __forceinline__ void storeN(int32_t *out, uint8_t *mout, int p, int t_cap, const int32_t *t)
{
    if (p + N <= t_cap) {
        int i = 0;
#pragma unroll
        for (; i + 4 <= N; i += 4) {
            int4v_a4 v = {t[i], t[i + 1], t[i + 2], t[i + 3]};
            *reinterpret_cast<int4v_a4 *>(out + p + i) = v;
            if (mout) *reinterpret_cast<u32_a1 *>(mout + p + i) = 0x01010101u;
        }
        if (i + 2 <= N) {
            int2v_a4 v = {t[i], t[i + 1]};
            *reinterpret_cast<int2v_a4 *>(out + p + i) = v;
            if (mout) *reinterpret_cast<u16_a1 *>(mout + p + i) = (uint16_t)0x0101u;
            i += 2;
        }
        if (i < N) {
            out[p + i] = t[i];
            if (mout) mout[p + i] = 1;
        }
    } else {
#pragma unroll
        for (int i = 0; i < N; ++i) store1(out, mout, p + i, t_cap, t[i]);
    }
}

template <int K, bool LUT4_LDS, bool CHARS>
__global__ __launch_bounds__(kKmerThreads) void kmer_rows_kernel(
    KmerArgs a, const uint8_t *__restrict__ bytes, const int64_t *__restrict__ offsets,
    int64_t n_rows, int64_t t_cap, int64_t fill_to, int32_t *__restrict__ ids,
    uint8_t *__restrict__ mask, int32_t *__restrict__ lengths, int32_t *__restrict__ status,
    int32_t *__restrict__ max_len)
{
    constexpr uint32_t POW4 = 1u << (2 * K);
    __shared__ uint32_t s_dig[256];
    __shared__ int32_t s_single[256];
    __shared__ int32_t s_lut4[LUT4_LDS ? POW4 : 1];
    __shared__ int32_t s_spell[256];     // token a byte is spelled with inside a non-plain window

    for (int i = threadIdx.x; i < 256; i += kKmerThreads) {
        const int d = a.digit[i];
        s_dig[i] = d < 0 ? kDigBad : (d >= 4 ? kDigN : (uint32_t)d);
        s_single[i] = a.single[i];
        // a byte outside the alphabet counts as N inside a window
        s_spell[i] = a.single[(int)"ACGTN"[d < 0 || d > 4 ? 4 : d]];
    }
    if (LUT4_LDS)
        for (uint32_t i = threadIdx.x; i < POW4; i += kKmerThreads) s_lut4[i] = a.lut4[i];
    __syncthreads();          // the only workgroup barrier: from here on every wave runs alone

    const int lane = threadIdx.x & 63;
    const int64_t wave = (int64_t)blockIdx.x * (kKmerThreads / 64) + (threadIdx.x >> 6);
    const int64_t n_waves = (int64_t)gridDim.x * (kKmerThreads / 64);
    int64_t wave_max = 0;

    for (int64_t row = wave; row < n_rows; row += n_waves) {
        const int64_t row_start = offsets[row];
        // positions inside a row are 32-bit: a row is shorter than 2^31 bytes
        const int len = (int)(offsets[row + 1] - row_start);
        const int full = len / K;
        const int n_units = full + (len - full * K);
        const uint8_t *src = bytes + row_start;
        int32_t *out = ids + row * t_cap;
        uint8_t *mout = mask ? mask + row * t_cap : nullptr;
        const int cap = t_cap > INT_MAX ? INT_MAX : (int)t_cap;
        int running = 0;
        int32_t my_status = 0;

        // software pipeline: the bytes of the next step are requested before this step is decoded
        uint32_t wn[K];
#pragma unroll
        for (int i = 0; i < K; ++i) wn[i] = 0;             // byte 0 is never a base
        if (lane * kUnitsPerLane + kUnitsPerLane <= full) memcpy(wn, src + lane * kUnitsPerLane * K, 4 * K);

        for (int u0 = 0; u0 < n_units; u0 += kWaveUnits) {
            const int ub = u0 + lane * kUnitsPerLane;
            const bool lane_full = ub + kUnitsPerLane <= full;     // 4 whole windows
            const bool empty = ub >= n_units;
            uint32_t w[K];
#pragma unroll
            for (int i = 0; i < K; ++i) { w[i] = wn[i]; wn[i] = 0; }
            if (ub + kWaveUnits + kUnitsPerLane <= full)            // 4 windows = 4K bytes, unaligned
                memcpy(wn, src + (ub + kWaveUnits) * K, 4 * K);
            // digit of byte bi of this lane (LDS lookup)
            auto digit_of = [&](int bi) -> uint32_t { return s_dig[(w[bi >> 2] >> (8 * (bi & 3))) & 255u]; };
            uint32_t code[kUnitsPerLane];
#pragma unroll
            for (int j = 0; j < kUnitsPerLane; ++j) {
                uint32_t c = 0;
#pragma unroll
                for (int i = 0; i < K; ++i) c = (c << 2) + digit_of(j * K + i);
                code[j] = c;
            }
            int32_t t[kUnitsPerLane];
#pragma unroll
            for (int j = 0; j < kUnitsPerLane; ++j) {
                const uint32_t idx = code[j] & (POW4 - 1);
                t[j] = LUT4_LDS ? s_lut4[idx] : a.lut4[idx];
            }
            const uint32_t any_flag = code[0] | code[1] | code[2] | code[3];
            const bool fast = lane_full && any_flag < POW4 && (t[0] | t[1] | t[2] | t[3]) >= 0;
            const uint64_t fast_mask = __ballot(fast);
            const uint64_t rest_mask = __ballot(!fast && !empty);

            if (rest_mask == 0) {
                // every lane is plain or past the end: positions are known without a scan
                const int p = running + lane * kUnitsPerLane;
                if (fast) {
                    if (p + 4 <= cap) {
                        store4(out, mout, p, t);
                    } else {
#pragma unroll
                        for (int j = 0; j < kUnitsPerLane; ++j) store1(out, mout, p + j, cap, t[j]);
                    }
                }
                running += kUnitsPerLane * (int)__popcll(fast_mask);
                continue;
            }

            // ---- step with exceptions ----
            // per unit: cnt = number of tokens; ex/ey = entry of a window that is not plain
            int32_t cnt[kUnitsPerLane], ex[kUnitsPerLane], ey[kUnitsPerLane];
            uint32_t lane_cnt = 0;
            if (lane_full) {
#pragma unroll
                for (int j = 0; j < kUnitsPerLane; ++j) {
                    ex[j] = 0; ey[j] = 0;
                    if (code[j] < POW4 && t[j] >= 0) {
                        cnt[j] = 1;
                    } else if (CHARS) {
                        cnt[j] = K;
                    } else {
                        int c5 = 0;
#pragma unroll
                        for (int i = 0; i < K; ++i) {
                            const uint32_t v = digit_of(j * K + i);
                            c5 = c5 * 5 + ((v & (kDigN | kDigBad)) ? 4 : (int)v);
                        }
                        const int2 e = a.entry[c5];
                        ex[j] = e.x; ey[j] = e.y;
                        cnt[j] = e.x >= 0 ? 1 : (e.x == INT_MIN ? 1 : -e.x);
                        if (e.x == INT_MIN) my_status |= DNATOK_ROW_MISSING_KMER;
                    }
                    if ((code[j] >> 17) != 0) {
                        // some digit may carry the foreign-byte flag (bit 17, shifted left by 0..2(K-1))
                        bool bad = false;
#pragma unroll
                        for (int i = 0; i < K; ++i) bad = bad || (digit_of(j * K + i) & kDigBad);
                        if (bad) my_status |= DNATOK_ROW_INVALID_BYTE;
                    }
                    lane_cnt += (uint32_t)cnt[j];
                }
            } else if (!empty) {
                // the ragged end of the row: whole windows first, then single characters
#pragma unroll 1
                for (int j = 0; j < kUnitsPerLane; ++j) {
                    const int u = ub + j;
                    int n = 0;
                    if (u < full) {
                        uint32_t c = 0;
                        int c5 = 0;
#pragma unroll
                        for (int i = 0; i < K; ++i) {
                            const uint32_t v = s_dig[src[u * K + i]];
                            c = (c << 2) + v;
                            if (v & kDigBad) my_status |= DNATOK_ROW_INVALID_BYTE;
                            c5 = c5 * 5 + ((v & (kDigN | kDigBad)) ? 4 : (int)v);
                        }
                        int32_t id = -1;
                        if (c < POW4) id = LUT4_LDS ? s_lut4[c] : a.lut4[c];
                        if (id >= 0) {
                            n = 1;
                        } else {
                            const int2 e = a.entry[c5];
                            n = e.x >= 0 ? 1 : (e.x == INT_MIN ? 1 : -e.x);
                            if (e.x == INT_MIN) my_status |= DNATOK_ROW_MISSING_KMER;
                        }
                    } else if (u < n_units) {
                        n = 1;
                    }
                    lane_cnt += (uint32_t)n;
                }
            }

            const uint32_t inc = wave_inclusive_sum_u32(lane_cnt);
            const uint32_t step_total = __builtin_amdgcn_readlane(inc, 63);
            int p = running + (int)(inc - lane_cnt);

            if (fast) {
                if (p + 4 <= cap) {
                    store4(out, mout, p, t);
                } else {
#pragma unroll
                    for (int j = 0; j < kUnitsPerLane; ++j) store1(out, mout, p + j, cap, t[j]);
                }
            } else if (lane_full) {
#pragma unroll
                for (int j = 0; j < kUnitsPerLane; ++j) {
                    if (code[j] < POW4 && t[j] >= 0) {
                        store1(out, mout, p, cap, t[j]);
                        ++p;
                    } else if (CHARS) {
                        int32_t sp[K];
#pragma unroll
                        for (int i = 0; i < K; ++i) {
                            const int bi = j * K + i;
                            sp[i] = s_spell[(w[bi >> 2] >> (8 * (bi & 3))) & 255u];
                        }
                        storeN<K>(out, mout, p, cap, sp);
                        p += K;
                    } else if (ex[j] >= 0) {
                        store1(out, mout, p, cap, ex[j]);
                        ++p;
                    } else if (ex[j] == INT_MIN) {
                        store1(out, mout, p, cap, a.missing_id);
                        ++p;
                    } else {
                        for (int e = 0; e < -ex[j]; ++e) store1(out, mout, p + e, cap, a.flat[ey[j] + e]);
                        p += -ex[j];
                    }
                }
            } else if (!empty) {
#pragma unroll 1
                for (int j = 0; j < kUnitsPerLane; ++j) {
                    const int u = ub + j;
                    if (u < full) {
                        uint32_t c = 0;
                        int c5 = 0;
#pragma unroll
                        for (int i = 0; i < K; ++i) {
                            const uint32_t v = s_dig[src[u * K + i]];
                            c = (c << 2) + v;
                            c5 = c5 * 5 + ((v & (kDigN | kDigBad)) ? 4 : (int)v);
                        }
                        int32_t id = -1;
                        if (c < POW4) id = LUT4_LDS ? s_lut4[c] : a.lut4[c];
                        if (id >= 0) {
                            store1(out, mout, p, cap, id);
                            ++p;
                        } else {
                            const int2 e = a.entry[c5];
                            if (e.x >= 0 || e.x == INT_MIN) {
                                store1(out, mout, p, cap, e.x >= 0 ? e.x : a.missing_id);
                                ++p;
                            } else {
                                for (int q = 0; q < -e.x; ++q) store1(out, mout, p + q, cap, a.flat[e.y + q]);
                                p += -e.x;
                            }
                        }
                    } else if (u < n_units) {
                        store1(out, mout, p, cap, s_single[src[full * K + (u - full)]]);
                        ++p;
                    }
                }
            }
            running += (int)step_total;
        }

        const int64_t stored = running < cap ? running : cap;
        int32_t st = 0;
        if (__ballot(my_status & DNATOK_ROW_INVALID_BYTE)) st |= DNATOK_ROW_INVALID_BYTE;
        if (__ballot(my_status & DNATOK_ROW_MISSING_KMER)) st |= DNATOK_ROW_MISSING_KMER;
        if (running > t_cap) st |= DNATOK_ROW_TRUNCATED;
        if (lane == 0) {
            lengths[row] = (int32_t)running;
            if (status) status[row] = st;
        }
        if (stored > wave_max) wave_max = stored;
        if (fill_to > 0) {
            for (int64_t p = stored + lane; p < fill_to; p += 64) {
                out[p] = a.pad_id;
                if (mout) mout[p] = 0;
            }
        }
    }
    // one atomic per wave at most, skipped when another wave already published a larger value
    if (max_len && lane == 0 && wave_max > 0 &&
        (int64_t)__builtin_nontemporal_load(max_len) < wave_max)
        atomicMax(max_len, (int32_t)wave_max);
}

// Pads every row from its stored length up to the batch maximum found on the device.
// One wave per row.
__global__ __launch_bounds__(256) void pad_to_max_kernel(
    int32_t *__restrict__ ids, uint8_t *__restrict__ mask, const int32_t *__restrict__ lengths,
    int64_t n_rows, int64_t t_cap, const int32_t *__restrict__ max_len, int32_t pad_id)
{
    const int64_t fill = *max_len;
    const int lane = threadIdx.x & 63;
    const int64_t wave = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    const int64_t n_waves = (int64_t)gridDim.x * (blockDim.x >> 6);
    for (int64_t row = wave; row < n_rows; row += n_waves) {
        int64_t len = lengths[row];
        if (len > t_cap) len = t_cap;
        if (len < 0) len = 0;
        for (int64_t p = len + lane; p < fill; p += 64) {
            ids[row * t_cap + p] = pad_id;
            if (mask) mask[row * t_cap + p] = 0;
        }
    }
}

int launch_pad_to_max(int32_t *ids, uint8_t *mask, const int32_t *lengths, int64_t n_rows,
                      int64_t t_cap, const int32_t *max_len, int32_t pad_id, hipStream_t s)
{
    int64_t blocks = (n_rows + 3) / 4;
    if (blocks > 256 * 16) blocks = 256 * 16;
    if (blocks < 1) blocks = 1;
    pad_to_max_kernel<<<(int)blocks, 256, 0, s>>>(ids, mask, lengths, n_rows, t_cap, max_len, pad_id);
    DNATOK_HIP_TRY(hipGetLastError());
    return DNATOK_OK;
}

int launch_zero_i32(int32_t *p, hipStream_t s)
{
    zero_i32_kernel<<<1, 1, 0, s>>>(p);
    DNATOK_HIP_TRY(hipGetLastError());
    return DNATOK_OK;
}

}  // namespace dnatok

using namespace dnatok;

extern "C" int dnatok_kmer_table_create(int k, const int8_t *digit_h, const int32_t *kmer_lut_h,
                                        const int32_t *exp_off_h, const int32_t *exp_len_h,
                                        const int32_t *exp_flat_h, int64_t n_flat,
                                        const int32_t *single_h, int32_t pad_id, int32_t missing_id,
                                        dnatok_kmer_t **out)
{
    DNATOK_REQUIRE(digit_h && kmer_lut_h && single_h && out, DNATOK_E_INVALID,
                   "dnatok_kmer_table_create: null argument");
    DNATOK_REQUIRE(k >= 2 && k <= 8, DNATOK_E_INVALID, "dnatok_kmer_table_create: k=%d outside 2..8", k);
    const bool has_exp = exp_off_h && exp_len_h && exp_flat_h && n_flat > 0;
    int64_t pow4 = 1, pow5 = 1;
    for (int i = 0; i < k; ++i) { pow4 *= 4; pow5 *= 5; }
    if (has_exp) {
        for (int64_t c = 0; c < pow5; ++c) {
            DNATOK_REQUIRE(exp_len_h[c] >= 0 && exp_off_h[c] >= 0 &&
                               (int64_t)exp_off_h[c] + exp_len_h[c] <= n_flat,
                           DNATOK_E_INVALID, "dnatok_kmer_table_create: expansion of window %lld out of range",
                           (long long)c);
        }
    }
    // lut4[c4]: re-index the ACGT-only windows from base 5 to base 4
    std::vector<int32_t> lut4(pow4);
    for (int64_t c4 = 0; c4 < pow4; ++c4) {
        int64_t c5 = 0;
        for (int i = k - 1; i >= 0; --i) c5 = c5 * 5 + ((c4 >> (2 * i)) & 3);
        lut4[c4] = kmer_lut_h[c5];
    }
    // entry[c5]: one 8-byte record per window, and whether every window without an id is
    // spelled by its own characters (then the kernel never reads entry / flat)
    std::vector<int2> entry(pow5);
    const char alphabet[6] = "ACGTN";
    bool chars_mode = true;
    for (int64_t c = 0; c < pow5; ++c) {
        if (kmer_lut_h[c] >= 0) {
            entry[c] = int2{kmer_lut_h[c], 0};
            bool has_n = false;
            int64_t v = c;
            for (int i = 0; i < k; ++i, v /= 5) has_n = has_n || (v % 5 == 4);
            if (has_n) chars_mode = false;             // an N window with an id of its own
        } else if (has_exp && exp_len_h[c] > 0) {
            entry[c] = int2{-exp_len_h[c], exp_off_h[c]};
            bool spelled = exp_len_h[c] == k;
            int64_t v = c;
            for (int i = k - 1; i >= 0 && spelled; --i, v /= 5)
                spelled = exp_flat_h[exp_off_h[c] + i] == single_h[(int)alphabet[v % 5]];
            if (!spelled) chars_mode = false;
        } else {
            entry[c] = int2{INT_MIN, 0};
            chars_mode = false;
        }
    }
    auto up = [](size_t v) { return (v + 255) & ~(size_t)255; };
    const size_t o_digit = 0;
    const size_t o_single = up(o_digit + 256);
    const size_t o_lut4 = up(o_single + 256 * 4);
    const size_t o_entry = up(o_lut4 + pow4 * 4);
    const size_t o_flat = up(o_entry + pow5 * sizeof(int2));
    const size_t bytes = up(o_flat + (has_exp ? n_flat * 4 : 0)) + 256;
    std::vector<uint8_t> host(bytes, 0);
    memcpy(&host[o_digit], digit_h, 256);
    memcpy(&host[o_single], single_h, 256 * 4);
    memcpy(&host[o_lut4], lut4.data(), pow4 * 4);
    memcpy(&host[o_entry], entry.data(), pow5 * sizeof(int2));
    if (has_exp) memcpy(&host[o_flat], exp_flat_h, n_flat * 4);
    void *blob = nullptr;
    hipError_t e = hipMalloc(&blob, bytes);
    if (e == hipSuccess) e = hipMemcpy(blob, host.data(), bytes, hipMemcpyHostToDevice);
    if (e != hipSuccess) {
        set_error("dnatok_kmer_table_create: %s", hipGetErrorString(e));
        if (blob) (void)hipFree(blob);
        return DNATOK_E_HIP;
    }
    dnatok_kmer_table *t = new dnatok_kmer_table();
    uint8_t *b = (uint8_t *)blob;
    t->k = k; t->pow4 = pow4; t->pow5 = pow5; t->pad_id = pad_id; t->missing_id = missing_id;
    t->chars_mode = chars_mode; t->blob = blob;
    t->digit = (int8_t *)(b + o_digit);
    t->single = (int32_t *)(b + o_single);
    t->lut4 = (int32_t *)(b + o_lut4);
    t->entry = (int2 *)(b + o_entry);
    t->flat = (int32_t *)(b + o_flat);
    *out = t;
    return DNATOK_OK;
}

extern "C" void dnatok_kmer_table_destroy(dnatok_kmer_t *t)
{
    if (!t) return;
    if (t->blob) (void)hipFree(t->blob);
    delete t;
}

extern "C" int dnatok_kmer_encode_padded(const dnatok_kmer_t *t, const uint8_t *bytes,
                                         const int64_t *offsets, int64_t n_rows, int64_t t_cap,
                                         int64_t fill_to, int32_t *ids, uint8_t *mask,
                                         int32_t *lengths, int32_t *status, int32_t *max_len,
                                         void *stream)
{
    DNATOK_REQUIRE(t && offsets && ids && lengths, DNATOK_E_INVALID,
                   "dnatok_kmer_encode_padded: null argument");
    DNATOK_REQUIRE(n_rows >= 0 && t_cap >= 0 && fill_to >= 0 && fill_to <= t_cap, DNATOK_E_INVALID,
                   "dnatok_kmer_encode_padded: need 0 <= fill_to <= t_cap");
    DNATOK_REQUIRE(fill_to > 0 || max_len, DNATOK_E_INVALID,
                   "dnatok_kmer_encode_padded: fill_to = 0 needs max_len");
    if (n_rows == 0) return DNATOK_OK;
    hipStream_t s = (hipStream_t)stream;
    if (max_len) {
        int rc = launch_zero_i32(max_len, s);
        if (rc) return rc;
    }
    KmerArgs a{t->digit, t->single, t->lut4, t->entry, t->flat, t->pad_id, t->missing_id};
    // persistent waves: the tables are staged into LDS once per workgroup, rows are dealt
    // round-robin to waves
    const int64_t want = (n_rows + kKmerThreads / 64 - 1) / (kKmerThreads / 64);
#define LAUNCH2(KK, L, C)                                                                         \
    do {                                                                                          \
        static const int resident = resident_workgroups(kmer_rows_kernel<KK, L, C>, kKmerThreads, 0, 4); \
        const int64_t grid = want < resident ? want : resident;                                   \
        kmer_rows_kernel<KK, L, C><<<(int)grid, kKmerThreads, 0, s>>>(                            \
            a, bytes, offsets, n_rows, t_cap, fill_to, ids, mask, lengths, status, max_len);      \
    } while (0)
#define LAUNCH(KK, L)                                                                             \
    do {                                                                                          \
        if (t->chars_mode) LAUNCH2(KK, L, true); else LAUNCH2(KK, L, false);                      \
    } while (0)
    switch (t->k) {
        case 2: LAUNCH(2, true); break;
        case 3: LAUNCH(3, true); break;
        case 4: LAUNCH(4, true); break;
        case 5: LAUNCH(5, true); break;
        case 6: LAUNCH(6, true); break;
        case 7: LAUNCH(7, false); break;
        default: LAUNCH(8, false); break;
    }
#undef LAUNCH
#undef LAUNCH2
    DNATOK_HIP_TRY(hipGetLastError());
    if (fill_to == 0) return launch_pad_to_max(ids, mask, lengths, n_rows, t_cap, max_len, t->pad_id, s);
    return DNATOK_OK;
}
