// Non-overlapping k-mer encoder with per-window fallback, tail handling, padding and mask.
//
// One workgroup walks one row in tiles of 1024 units (a unit is a k-base window, or one of
// the trailing len % k characters).  Each lane owns 4 consecutive units: it loads its 4k
// bytes, turns them into base-5 digits through an LDS digit table, and looks the window up
// in an LDS table of the 4^k N-free windows; a window holding N (or a byte outside the
// alphabet) goes through the global 5^k table and, when that entry is -1, is spelled out
// from the expansion lists.  Unit token counts are prefix-summed across the workgroup
// (wave64 scan + LDS carry), so every lane knows where its tokens land and a lane whose 4
// windows are plain writes one aligned 16-byte store.  Traffic: 1 byte read per base,
// 5 bytes written per token.
#include "common.hpp"

#include <string.h>
#include <vector>

struct dnatok_kmer_table {
    int k;
    int64_t pow4, pow5;
    int32_t pad_id, missing_id;
    int has_exp;
    void *blob;              // one device allocation holding all tables
    int8_t *digit;           // [256]
    int32_t *single;         // [256]
    int32_t *lut4;           // [4^k]  id of an ACGT-only window, or -1
    int32_t *lut5;           // [5^k]
    int32_t *exp_off, *exp_len, *exp_flat;
};

namespace dnatok {

struct KmerArgs {
    const int8_t *digit;
    const int32_t *single, *lut4, *lut5, *exp_off, *exp_len, *exp_flat;
    int32_t pad_id, missing_id;
};

constexpr int kKmerThreads = 256;
constexpr int kUnitsPerLane = 4;
constexpr int kTileUnits = kKmerThreads * kUnitsPerLane;

typedef int32_t int4v __attribute__((ext_vector_type(4)));

__global__ void zero_i32_kernel(int32_t *p) { *p = 0; }

// Exclusive prefix sum of one value per thread over the workgroup; total in *total_out.
__device__ __forceinline__ uint32_t block_exclusive_sum(uint32_t v, uint32_t *wave_tot, uint32_t *total_out)
{
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const uint32_t inc = wave_inclusive_sum_u32(v);
    if (lane == 63) wave_tot[wv] = inc;
    __syncthreads();
    uint32_t carry = 0, total = 0;
#pragma unroll
    for (int i = 0; i < kKmerThreads / 64; ++i) {
        const uint32_t t = wave_tot[i];
        if (i < wv) carry += t;
        total += t;
    }
    __syncthreads();   // wave_tot is reused by the next tile
    *total_out = total;
    return carry + inc - v;
}

template <int K, bool LUT4_LDS>
__global__ __launch_bounds__(kKmerThreads) void kmer_rows_kernel(
    KmerArgs a, const uint8_t *__restrict__ bytes, const int64_t *__restrict__ offsets,
    int64_t n_rows, int64_t t_cap, int64_t fill_to, int32_t *__restrict__ ids,
    uint8_t *__restrict__ mask, int32_t *__restrict__ lengths, int32_t *__restrict__ status,
    int32_t *__restrict__ max_len)
{
    constexpr int POW4 = 1 << (2 * K);
    __shared__ int8_t s_digit[256];
    __shared__ int32_t s_single[256];
    __shared__ int32_t s_lut4[LUT4_LDS ? POW4 : 1];
    __shared__ uint32_t s_wave_tot[kKmerThreads / 64];
    __shared__ int32_t s_status;

    s_digit[threadIdx.x] = a.digit[threadIdx.x];
    s_single[threadIdx.x] = a.single[threadIdx.x];
    if (LUT4_LDS)
        for (int i = threadIdx.x; i < POW4; i += kKmerThreads) s_lut4[i] = a.lut4[i];
    if (threadIdx.x == 0) s_status = 0;
    __syncthreads();

    const bool ids_aligned = (((uintptr_t)ids & 15) == 0) && (t_cap % 4 == 0);
    const bool mask_aligned = mask && (((uintptr_t)mask & 3) == 0) && (t_cap % 4 == 0);

    for (int64_t row = blockIdx.x; row < n_rows; row += gridDim.x) {
        const int64_t row_start = offsets[row];
        const int64_t len = offsets[row + 1] - row_start;
        const int64_t full = len / K;
        const int64_t n_units = full + (len - full * K);
        const uint8_t *src = bytes + row_start;
        int32_t *out = ids + row * t_cap;
        uint8_t *mout = mask ? mask + row * t_cap : nullptr;
        int64_t running = 0;
        int32_t my_status = 0;

        for (int64_t u0 = 0; u0 < n_units; u0 += kTileUnits) {
            const int64_t ub = u0 + (int64_t)threadIdx.x * kUnitsPerLane;
            int32_t tok[kUnitsPerLane];     // the unit's token when cnt == 1
            int32_t cnt[kUnitsPerLane];     // tokens the unit produces
            int32_t code5[kUnitsPerLane];   // window code for units that expand
            uint32_t lane_cnt = 0;

            uint8_t ch[kUnitsPerLane * K];
            if (ub + kUnitsPerLane <= full) {
                uint32_t w[K];
                memcpy(w, src + ub * K, 4 * K);           // 4 windows = 4K bytes, unaligned
#pragma unroll
                for (int i = 0; i < kUnitsPerLane * K; ++i)
                    ch[i] = (uint8_t)((w[i >> 2] >> (8 * (i & 3))) & 255u);
            } else {
#pragma unroll
                for (int j = 0; j < kUnitsPerLane; ++j) {
                    const int64_t u = ub + j;
#pragma unroll
                    for (int i = 0; i < K; ++i)
                        ch[j * K + i] = (u < full) ? src[u * K + i] : (uint8_t)0;
                }
            }
#pragma unroll
            for (int j = 0; j < kUnitsPerLane; ++j) {
                const int64_t u = ub + j;
                tok[j] = 0; cnt[j] = 0; code5[j] = -1;
                if (u < full) {
                    int c4 = 0, c5 = 0;
                    bool plain = true;
#pragma unroll
                    for (int i = 0; i < K; ++i) {
                        int d = s_digit[ch[j * K + i]];
                        if (d < 0) { d = 4; my_status |= DNATOK_ROW_INVALID_BYTE; }
                        plain = plain && (d < 4);
                        c4 = (c4 << 2) | (d & 3);
                        c5 = c5 * 5 + d;
                    }
                    int32_t id = -1;
                    if (plain) id = LUT4_LDS ? s_lut4[c4] : a.lut4[c4];
                    if (id < 0) id = a.lut5[c5];
                    if (id >= 0) {
                        tok[j] = id; cnt[j] = 1;
                    } else if (a.exp_len && a.exp_len[c5] > 0) {
                        cnt[j] = a.exp_len[c5]; code5[j] = c5;
                    } else {
                        tok[j] = a.missing_id; cnt[j] = 1; my_status |= DNATOK_ROW_MISSING_KMER;
                    }
                } else if (u < n_units) {
                    tok[j] = s_single[src[full * K + (u - full)]];
                    cnt[j] = 1;
                }
                lane_cnt += (uint32_t)cnt[j];
            }

            uint32_t tile_total;
            const uint32_t off = block_exclusive_sum(lane_cnt, s_wave_tot, &tile_total);
            int64_t p = running + off;
            if (lane_cnt == kUnitsPerLane && code5[0] < 0 && code5[1] < 0 && code5[2] < 0 &&
                code5[3] < 0 && (p & 3) == 0 && p + 4 <= t_cap && ids_aligned) {
                int4v v = {tok[0], tok[1], tok[2], tok[3]};
                __builtin_nontemporal_store(v, reinterpret_cast<int4v *>(out + p));
                if (mask_aligned)
                    __builtin_nontemporal_store(0x01010101u, reinterpret_cast<uint32_t *>(mout + p));
                else if (mout) { mout[p] = 1; mout[p + 1] = 1; mout[p + 2] = 1; mout[p + 3] = 1; }
            } else {
#pragma unroll
                for (int j = 0; j < kUnitsPerLane; ++j) {
                    if (code5[j] < 0) {
                        if (cnt[j] == 1) {
                            if (p < t_cap) { out[p] = tok[j]; if (mout) mout[p] = 1; }
                            ++p;
                        }
                    } else {
                        const int32_t eo = a.exp_off[code5[j]];
                        for (int e = 0; e < cnt[j]; ++e) {
                            if (p < t_cap) { out[p] = a.exp_flat[eo + e]; if (mout) mout[p] = 1; }
                            ++p;
                        }
                    }
                }
            }
            running += tile_total;
        }

        if (my_status) atomicOr(&s_status, my_status);
        __syncthreads();
        const int64_t stored = running < t_cap ? running : t_cap;
        if (threadIdx.x == 0) {
            int32_t st = s_status;
            if (running > t_cap) st |= DNATOK_ROW_TRUNCATED;
            lengths[row] = (int32_t)running;
            if (status) status[row] = st;
            if (max_len) atomicMax(max_len, (int32_t)stored);
            s_status = 0;
        }
        if (fill_to > 0) {
            for (int64_t p = stored + threadIdx.x; p < fill_to; p += kKmerThreads) {
                out[p] = a.pad_id;
                if (mout) mout[p] = 0;
            }
        }
        __syncthreads();
    }
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
    auto up = [](size_t v) { return (v + 255) & ~(size_t)255; };
    const size_t o_digit = 0;
    const size_t o_single = up(o_digit + 256);
    const size_t o_lut4 = up(o_single + 256 * 4);
    const size_t o_lut5 = up(o_lut4 + pow4 * 4);
    const size_t o_eoff = up(o_lut5 + pow5 * 4);
    const size_t o_elen = up(o_eoff + (has_exp ? pow5 * 4 : 0));
    const size_t o_flat = up(o_elen + (has_exp ? pow5 * 4 : 0));
    const size_t bytes = up(o_flat + (has_exp ? n_flat * 4 : 0)) + 256;
    std::vector<uint8_t> host(bytes, 0);
    memcpy(&host[o_digit], digit_h, 256);
    memcpy(&host[o_single], single_h, 256 * 4);
    memcpy(&host[o_lut4], lut4.data(), pow4 * 4);
    memcpy(&host[o_lut5], kmer_lut_h, pow5 * 4);
    if (has_exp) {
        memcpy(&host[o_eoff], exp_off_h, pow5 * 4);
        memcpy(&host[o_elen], exp_len_h, pow5 * 4);
        memcpy(&host[o_flat], exp_flat_h, n_flat * 4);
    }
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
    t->has_exp = has_exp; t->blob = blob;
    t->digit = (int8_t *)(b + o_digit);
    t->single = (int32_t *)(b + o_single);
    t->lut4 = (int32_t *)(b + o_lut4);
    t->lut5 = (int32_t *)(b + o_lut5);
    t->exp_off = has_exp ? (int32_t *)(b + o_eoff) : nullptr;
    t->exp_len = has_exp ? (int32_t *)(b + o_elen) : nullptr;
    t->exp_flat = has_exp ? (int32_t *)(b + o_flat) : nullptr;
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
    KmerArgs a{t->digit, t->single, t->lut4, t->lut5, t->exp_off, t->exp_len, t->exp_flat,
               t->pad_id, t->missing_id};
    int64_t grid = n_rows < 256 * 64 ? n_rows : 256 * 64;
#define LAUNCH(KK, L)                                                                            \
    kmer_rows_kernel<KK, L><<<(int)grid, kKmerThreads, 0, s>>>(a, bytes, offsets, n_rows, t_cap, \
                                                               fill_to, ids, mask, lengths, status, max_len)
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
    DNATOK_HIP_TRY(hipGetLastError());
    if (fill_to == 0) return launch_pad_to_max(ids, mask, lengths, n_rows, t_cap, max_len, t->pad_id, s);
    return DNATOK_OK;
}
