// Memory-only kernels for measurements: what the machine gives a kernel of a given access shape
// when it does no arithmetic.  bench.py reports them beside the encoders' figures; nothing else
// calls them.
#include "common.hpp"

namespace dnatok {
namespace {

typedef uint32_t dg_u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t dg_u32x2 __attribute__((ext_vector_type(2)));

// A workgroup copies contiguous tiles of 16 KB (four 16-byte loads per lane, then four stores),
// tiles dealt round robin: the fastest plain copy measured on this machine.
__global__ __launch_bounds__(256) void diag_copy_tiles_kernel(const dg_u32x4 *__restrict__ src,
                                                              dg_u32x4 *__restrict__ dst, size_t n16)
{
    constexpr size_t kTile = 4 * 256;
    const size_t n_tiles = n16 / kTile;
    for (size_t t = blockIdx.x; t < n_tiles; t += gridDim.x) {
        const size_t b = t * kTile + threadIdx.x;
        dg_u32x4 v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) v[u] = __builtin_nontemporal_load(src + b + u * 256);
#pragma unroll
        for (int u = 0; u < 4; ++u) __builtin_nontemporal_store(v[u], dst + b + u * 256);
    }
    // (the bytes past the last whole tile)
    for (size_t i = n_tiles * kTile + (size_t)blockIdx.x * 256 + threadIdx.x; i < n16; i += (size_t)gridDim.x * 256)
        dst[i] = src[i];
}

// The memory operations of kmer_rows_kernel for k = 6 on rows of plain bases, and nothing else:
// persistent workgroups of eight waves, a wave per row, the row in steps of 1536 bytes read as 24
// bytes per lane one step ahead, 256 ids (16 bytes per lane) and 256 mask bytes written per step,
// the cells from the row's last token up to fill_to written as padding.
__global__ __launch_bounds__(512) void diag_kmer_shape_kernel(const uint8_t *__restrict__ bytes,
                                                              const int64_t *__restrict__ offsets, int64_t n_rows,
                                                              int64_t t_cap, int64_t fill_to,
                                                              int32_t *__restrict__ ids, uint8_t *__restrict__ mask)
{
    const int lane = threadIdx.x & 63;
    const int64_t wave = (int64_t)blockIdx.x * 8 + (threadIdx.x >> 6);
    const int64_t n_waves = (int64_t)gridDim.x * 8;
    for (int64_t row = wave; row < n_rows; row += n_waves) {
        const int64_t start = offsets[row];
        const int len = (int)(offsets[row + 1] - start);
        const int n_cells = len / 6 < (int)t_cap ? len / 6 : (int)t_cap;
        const int n_fill = fill_to > n_cells ? (int)fill_to : n_cells;
        const __amdgpu_buffer_rsrc_t rs =
            __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t *>(bytes + start), (short)0, len, 0x00020000);
        const __amdgpu_buffer_rsrc_t ro = __builtin_amdgcn_make_buffer_rsrc(ids + row * t_cap, (short)0, n_fill * 4, 0x00020000);
        const __amdgpu_buffer_rsrc_t rm = __builtin_amdgcn_make_buffer_rsrc(mask + row * t_cap, (short)0, n_fill, 0x00020000);
        const int n_steps = (len + 1535) / 1536;
        dg_u32x4 a, na;
        dg_u32x2 b, nb;
        na = __builtin_amdgcn_raw_buffer_load_b128(rs, lane * 24, 0, 0);
        nb = __builtin_amdgcn_raw_buffer_load_b64(rs, lane * 24 + 16, 0, 0);
        for (int st = 0; st < n_steps; ++st) {
            a = na; b = nb;
            na = __builtin_amdgcn_raw_buffer_load_b128(rs, (st + 1) * 1536 + lane * 24, 0, 0);
            nb = __builtin_amdgcn_raw_buffer_load_b64(rs, (st + 1) * 1536 + lane * 24 + 16, 0, 0);
            const dg_u32x4 v = {a.x ^ b.x, a.y ^ b.y, a.z + b.x, a.w + b.y};
            __builtin_amdgcn_raw_buffer_store_b128(v, ro, st * 1024 + lane * 16, 0, 2);
            __builtin_amdgcn_raw_buffer_store_b32(0x01010101u, rm, st * 256 + lane * 4, 0, 2);
        }
        // padding: the descriptors end at fill_to, so whole groups are stored without a test
        for (int c = n_steps * 256 + lane * 4; c < n_fill; c += 256) {
            const dg_u32x4 z = {0, 0, 0, 0};
            __builtin_amdgcn_raw_buffer_store_b128(z, ro, c * 4, 0, 2);
            __builtin_amdgcn_raw_buffer_store_b32(0u, rm, c, 0, 2);
        }
    }
}

}  // namespace
}  // namespace dnatok

using namespace dnatok;

extern "C" int dnatok_diag_copy_tiles(const void *src, void *dst, size_t bytes, void *stream)
{
    DNATOK_REQUIRE(src && dst, DNATOK_E_INVALID, "dnatok_diag_copy_tiles: null argument");
    DNATOK_REQUIRE(bytes % 16 == 0 && ((uintptr_t)src & 15) == 0 && ((uintptr_t)dst & 15) == 0, DNATOK_E_INVALID,
                   "dnatok_diag_copy_tiles: buffers and size must be multiples of 16 bytes");
    if (bytes == 0) return DNATOK_OK;
    diag_copy_tiles_kernel<<<8192, 256, 0, (hipStream_t)stream>>>((const dg_u32x4 *)src, (dg_u32x4 *)dst, bytes / 16);
    DNATOK_HIP_TRY(hipGetLastError());
    return DNATOK_OK;
}

extern "C" int dnatok_diag_kmer_shape(const uint8_t *bytes, const int64_t *offsets, int64_t n_rows, int64_t t_cap,
                                      int64_t fill_to, int32_t *ids, uint8_t *mask, void *stream)
{
    DNATOK_REQUIRE(bytes && offsets && ids && mask, DNATOK_E_INVALID, "dnatok_diag_kmer_shape: null argument");
    DNATOK_REQUIRE(n_rows >= 0 && t_cap >= 0 && t_cap % 4 == 0 && fill_to <= t_cap && t_cap < (int64_t)1 << 28,
                   DNATOK_E_INVALID, "dnatok_diag_kmer_shape: need fill_to <= t_cap, t_cap a multiple of 4 below 2^28");
    DNATOK_REQUIRE(((uintptr_t)ids & 15) == 0, DNATOK_E_INVALID, "dnatok_diag_kmer_shape: ids must be 16-byte aligned");
    if (n_rows == 0) return DNATOK_OK;
    const int64_t want = (n_rows + 7) / 8;
    diag_kmer_shape_kernel<<<(int)(want < 512 ? want : 512), 512, 0, (hipStream_t)stream>>>(bytes, offsets, n_rows, t_cap,
                                                                                          fill_to, ids, mask);
    DNATOK_HIP_TRY(hipGetLastError());
    return DNATOK_OK;
}
