// Shared helpers of libdnatok_hip: error reporting and wave64 cross-lane primitives (gfx950).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/dnatok_hip.h"

namespace dnatok {

void set_error(const char *fmt, ...);

#define DNATOK_HIP_TRY(call)                                                           \
    do {                                                                               \
        hipError_t e__ = (call);                                                       \
        if (e__ != hipSuccess) {                                                       \
            dnatok::set_error("%s failed: %s", #call, hipGetErrorString(e__));         \
            return DNATOK_E_HIP;                                                       \
        }                                                                              \
    } while (0)

#define DNATOK_REQUIRE(cond, code, ...)                                                \
    do {                                                                               \
        if (!(cond)) {                                                                 \
            dnatok::set_error(__VA_ARGS__);                                            \
            return (code);                                                             \
        }                                                                              \
    } while (0)

constexpr int kWave = 64;

// Workgroups of `kernel` that are resident at once on the current device (all CUs), for
// persistent launches: a grid of exactly this size runs as one wave of workgroups.
template <typename Kernel>
inline int resident_workgroups(Kernel kernel, int block_threads, size_t dynamic_lds, int fallback_per_cu)
{
    int dev = 0, cus = 256, per_cu = 0;
    if (hipGetDevice(&dev) == hipSuccess) {
        int v = 0;
        if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0) cus = v;
    }
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, block_threads, dynamic_lds) != hipSuccess ||
        per_cu <= 0) {
        (void)hipGetLastError();
        per_cu = fallback_per_cu;
    }
    return cus * per_cu;
}

// ---- wave64 cross-lane primitives (DPP within rows of 16 lanes, readlane across rows) ----

template <int CTRL>
__device__ __forceinline__ uint32_t dpp_u32(uint32_t v)
{
    // bound_ctrl = false and old = v: lanes without a valid source keep their own value
    return (uint32_t)__builtin_amdgcn_update_dpp((int)v, (int)v, CTRL, 0xF, 0xF, false);
}

__device__ __forceinline__ uint32_t umin(uint32_t a, uint32_t b) { return a < b ? a : b; }

// Minimum over the 64 lanes, returned in every lane (wave-uniform).
__device__ __forceinline__ uint32_t wave_min_u32(uint32_t v)
{
    v = umin(v, dpp_u32<0xB1>(v));   // quad_perm [1,0,3,2]
    v = umin(v, dpp_u32<0x4E>(v));   // quad_perm [2,3,0,1]
    v = umin(v, dpp_u32<0x141>(v));  // row_half_mirror
    v = umin(v, dpp_u32<0x140>(v));  // row_mirror
    uint32_t r0 = __builtin_amdgcn_readlane(v, 0);
    uint32_t r1 = __builtin_amdgcn_readlane(v, 16);
    uint32_t r2 = __builtin_amdgcn_readlane(v, 32);
    uint32_t r3 = __builtin_amdgcn_readlane(v, 48);
    return umin(umin(r0, r1), umin(r2, r3));
}

// row_shr:N within each row of 16 lanes; lanes without a source read 0.
template <int N>
__device__ __forceinline__ uint32_t dpp_row_shr_zero(uint32_t v)
{
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x110 + N, 0xF, 0xF, true);
}

// Inclusive prefix sum over the 64 lanes: DPP scan inside each row of 16, then the three
// row totals are carried across with readlane.
__device__ __forceinline__ uint32_t wave_inclusive_sum_u32(uint32_t v)
{
    v += dpp_row_shr_zero<1>(v);
    v += dpp_row_shr_zero<2>(v);
    v += dpp_row_shr_zero<4>(v);
    v += dpp_row_shr_zero<8>(v);
    const uint32_t t0 = __builtin_amdgcn_readlane(v, 15);
    const uint32_t t1 = __builtin_amdgcn_readlane(v, 31);
    const uint32_t t2 = __builtin_amdgcn_readlane(v, 47);
    const uint32_t row = (threadIdx.x & 63) >> 4;
    uint32_t carry = 0;
    if (row >= 1) carry += t0;
    if (row >= 2) carry += t1;
    if (row >= 3) carry += t2;
    return v + carry;
}

__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v)
{
    return ~wave_min_u32(~v);
}

// ---- maximum over the workgroups of a launch, carried by atomics alone ----

constexpr int kTreeRows = 2048;          // workgroups of one launch that can take part
constexpr int kTreeWords = 1024;         // 512 + 128 + 32 + 8 + 2 + 1 words used, 8 KB per tree

// The longest row of a call without a padding pass (every row padded as far as any row can
// reach), found without a fence: nothing but atomics carries it.  Every workgroup adds its
// maximum + 1 into its 16-bit field of a 64-bit word shared by four workgroups; the atomic returns
// the fields of those that came before, so the workgroup that completes a word knows the maximum
// of its four, clears the word for the next call and carries the maximum one level up in the same
// way (a 4-ary tree, `tree` holds its words level by level).  Who completes the root writes
// max_len.  `mine` is the caller's value + 1 and `before` what its own atomicAdd at the lowest
// level returned (the caller issues that one itself, as early as it knows its value); one lane
// calls this.  (One counter and one atomicMax for 256 workgroups cost 3 us, two of them spent
// queueing at that one address.)
__device__ __forceinline__ void climb_max_tree(unsigned long long *tree, unsigned idx, unsigned n_here,
                                               unsigned long long mine, unsigned long long before,
                                               int32_t *__restrict__ max_len)
{
    unsigned long long *level = tree;
    // words this workgroup completed: cleared when it is done climbing, so that a level costs one
    // trip to memory (the add, whose answer is waited for) and not two
    unsigned long long *completed[8];
    int n_completed = 0;
    for (;;) {
        const unsigned long long all = before + (mine << (16 * (idx & 3)));
        const unsigned members = n_here - (idx & ~3u) < 4u ? n_here - (idx & ~3u) : 4u;
        unsigned arrived = 0;
        unsigned long long best = 0;
#pragma unroll
        for (int f = 0; f < 4; ++f) {
            const unsigned long long v = (all >> (16 * f)) & 0xFFFFull;
            arrived += v != 0;
            best = v > best ? v : best;
        }
        if (arrived < members) break;
        completed[n_completed++] = level + (idx >> 2);
        if (n_here <= 4) {
            *max_len = (int32_t)best - 1;
            break;
        }
        level += (n_here + 3) >> 2;
        n_here = (n_here + 3) >> 2;
        idx >>= 2;
        mine = best;
        before = atomicAdd(level + (idx >> 2), mine << (16 * (idx & 3)));
    }
    for (int i = 0; i < n_completed; ++i) atomicExch(completed[i], 0ull);
}

// The whole of it for a workgroup that knows its value (< 0xFFFF) only at its end: one lane calls
// this, every workgroup of the launch exactly once, gridDim.x <= kTreeRows.
__device__ __forceinline__ void publish_max(unsigned long long *tree, unsigned value, int32_t *__restrict__ max_len)
{
    const unsigned long long mine = (unsigned long long)value + 1ull;
    const unsigned long long before = atomicAdd(tree + (blockIdx.x >> 2), mine << (16 * (blockIdx.x & 3)));
    climb_max_tree(tree, blockIdx.x, gridDim.x, mine, before, max_len);
}

}  // namespace dnatok
