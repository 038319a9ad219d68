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

// Inclusive prefix sum over the 64 lanes.
__device__ __forceinline__ uint32_t wave_inclusive_sum_u32(uint32_t v)
{
    const int lane = threadIdx.x & 63;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        uint32_t o = __shfl_up(v, d, 64);
        if (lane >= d) v += o;
    }
    return v;
}

__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v)
{
    return ~wave_min_u32(~v);
}

}  // namespace dnatok
