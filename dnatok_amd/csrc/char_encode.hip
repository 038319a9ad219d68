// Single-nucleotide encoder: ids = table[byte], with padding and attention mask.
//
// HBM-bound streaming map: 1 byte read and 5 bytes written per base (int32 id + uint8 mask).
// The 256-entry table (and the optional first-column table) sit in LDS; DNA input touches
// five entries, so lanes either broadcast or hit distinct banks.  Each lane reads 4 bytes
// per step as one dword (a wave covers 256 contiguous bytes) and writes its 4 ids as one
// 16-byte store (a wave covers 1 KiB contiguous) and its 4 mask bytes as one dword.
#include "common.hpp"

#include <string.h>

namespace dnatok {

struct CharTableDev {
    int32_t lut[256];
    int32_t start[256];
};

}  // namespace dnatok

struct dnatok_char_table {
    dnatok::CharTableDev *dev;   // device copy
    int32_t pad_id;
    int has_start;
};

namespace dnatok {

constexpr int kCharThreads = 256;
constexpr int kCharSteps = 4;                                   // dwords per lane per tile
constexpr int kCharTile = kCharThreads * 4 * kCharSteps;        // 4096 bases per tile

typedef int32_t int4v __attribute__((ext_vector_type(4)));
typedef int32_t int4v_a4 __attribute__((ext_vector_type(4), aligned(4)));   // only the mask's 4-byte alignment is required

__device__ __forceinline__ int4v lookup4(const int32_t *lut, uint32_t w)
{
    int4v v;
    v.x = lut[w & 255u];
    v.y = lut[(w >> 8) & 255u];
    v.z = lut[(w >> 16) & 255u];
    v.w = lut[w >> 24];
    return v;
}

// Four ids of one of the output widths (uint8, int16, int32, int64) as one store.
template <typename OUT> struct Quad;
template <> struct Quad<uint8_t> { typedef uint32_t type; };
template <> struct Quad<int16_t> { typedef int16_t type __attribute__((ext_vector_type(4))); };
template <> struct Quad<int32_t> { typedef int4v type; };
template <> struct Quad<int64_t> { typedef int64_t type __attribute__((ext_vector_type(4))); };

template <typename OUT>
__device__ __forceinline__ typename Quad<OUT>::type make_quad(int4v v);
template <> __device__ __forceinline__ uint32_t make_quad<uint8_t>(int4v v)
{
    return (uint32_t)(v.x & 255) | ((uint32_t)(v.y & 255) << 8) | ((uint32_t)(v.z & 255) << 16) |
           ((uint32_t)v.w << 24);
}
template <> __device__ __forceinline__ Quad<int16_t>::type make_quad<int16_t>(int4v v)
{
    return Quad<int16_t>::type{(int16_t)v.x, (int16_t)v.y, (int16_t)v.z, (int16_t)v.w};
}
template <> __device__ __forceinline__ int4v make_quad<int32_t>(int4v v) { return v; }
template <> __device__ __forceinline__ Quad<int64_t>::type make_quad<int64_t>(int4v v)
{
    return Quad<int64_t>::type{(int64_t)v.x, (int64_t)v.y, (int64_t)v.z, (int64_t)v.w};
}

// Flat stream; requires bytes 4-byte aligned, ids 16-byte aligned, mask 4-byte aligned.
template <bool HAS_MASK, bool HAS_START>
__global__ __launch_bounds__(kCharThreads) void char_packed_kernel(
    const uint8_t *__restrict__ bytes, int64_t total, int64_t row_len,
    const CharTableDev *__restrict__ tab, int32_t *__restrict__ ids, uint8_t *__restrict__ mask)
{
    __shared__ int32_t lut[256];
    __shared__ int32_t start[256];
    lut[threadIdx.x] = tab->lut[threadIdx.x];
    if (HAS_START) start[threadIdx.x] = tab->start[threadIdx.x];
    __syncthreads();

    const int64_t n_tiles = (total + kCharTile - 1) / kCharTile;
    for (int64_t tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
        const int64_t base = tile * kCharTile + (int64_t)threadIdx.x * 4;
        uint32_t w[kCharSteps];
        if (tile * kCharTile + kCharTile <= total) {
#pragma unroll
            for (int s = 0; s < kCharSteps; ++s)
                w[s] = __builtin_nontemporal_load(
                    reinterpret_cast<const uint32_t *>(bytes + base + s * (kCharThreads * 4)));
#pragma unroll
            for (int s = 0; s < kCharSteps; ++s) {
                const int64_t i = base + s * (kCharThreads * 4);
                int4v v = lookup4(lut, w[s]);
                if (HAS_START) {
                    // rare path (separate first-column table): test each position exactly
                    const int64_t r = i % row_len;
                    if (r == 0) v.x = start[w[s] & 255u];
                    if ((r + 1) % row_len == 0) v.y = start[(w[s] >> 8) & 255u];
                    if ((r + 2) % row_len == 0) v.z = start[(w[s] >> 16) & 255u];
                    if ((r + 3) % row_len == 0) v.w = start[w[s] >> 24];
                }
                __builtin_nontemporal_store(v, reinterpret_cast<int4v *>(ids + i));
            }
            // the mask of a whole tile is 4096 ones: one 16-byte store per lane covers it
            if (HAS_MASK) {
                const int4v_a4 ones = {0x01010101, 0x01010101, 0x01010101, 0x01010101};
                __builtin_nontemporal_store(
                    ones, reinterpret_cast<int4v_a4 *>(mask + tile * kCharTile + (int64_t)threadIdx.x * 16));
            }
        } else {
            // last, partial tile: position by position
            for (int s = 0; s < kCharSteps; ++s) {
                for (int k = 0; k < 4; ++k) {
                    const int64_t i = base + s * (kCharThreads * 4) + k;
                    if (i < total) {
                        const uint8_t c = bytes[i];
                        const bool first = HAS_START && (i % row_len == 0);
                        ids[i] = first ? start[c] : lut[c];
                        if (HAS_MASK) mask[i] = 1;
                    }
                }
            }
        }
    }
}

// Ragged rows to a padded [n_rows, t_out] matrix.  One tile = 1024 output columns of one row.
// ALIGNED: t_out % 4 == 0, the ids base is aligned to four ids and the mask base to 4 bytes, so
// each lane stores its 4 columns with one store of four ids and one 4-byte store.  OUT is the
// width the ids are written in.
template <typename OUT, bool HAS_MASK, bool HAS_START, bool ALIGNED>
__global__ __launch_bounds__(kCharThreads) void char_padded_kernel(
    const uint8_t *__restrict__ bytes, const int64_t *__restrict__ offsets, int64_t n_rows,
    int64_t t_out, int64_t tiles_per_row, int pad_left, int32_t pad_id,
    const CharTableDev *__restrict__ tab, OUT *__restrict__ ids, uint8_t *__restrict__ mask)
{
    __shared__ int32_t lut[256];
    __shared__ int32_t start[256];
    lut[threadIdx.x] = tab->lut[threadIdx.x];
    if (HAS_START) start[threadIdx.x] = tab->start[threadIdx.x];
    __syncthreads();

    const int64_t n_tiles = n_rows * tiles_per_row;
    for (int64_t tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
        const int64_t b = tile / tiles_per_row;
        const int64_t col0 = (tile - b * tiles_per_row) * (kCharThreads * 4) + (int64_t)threadIdx.x * 4;
        if (col0 >= t_out) continue;
        const int64_t row_start = offsets[b];
        int64_t len = offsets[b + 1] - row_start;
        if (len > t_out) len = t_out;
        const int64_t shift = pad_left ? (t_out - len) : 0;   // first real column
        const uint8_t *src = bytes + row_start - shift;       // src[col] for shift <= col < shift+len
        int32_t v[4];
        uint32_t m = 0;
        if (col0 >= shift && col0 + 4 <= shift + len) {
            uint32_t w;
            memcpy(&w, src + col0, 4);                        // row starts are not aligned
            v[0] = lut[w & 255u]; v[1] = lut[(w >> 8) & 255u];
            v[2] = lut[(w >> 16) & 255u]; v[3] = lut[w >> 24];
            if (HAS_START && col0 == shift) v[0] = start[w & 255u];
            m = 0x01010101u;
        } else {
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const int64_t c = col0 + k;
                if (c >= shift && c < shift + len) {
                    const uint8_t ch = src[c];
                    v[k] = (HAS_START && c == shift) ? start[ch] : lut[ch];
                    m |= 1u << (8 * k);
                } else {
                    v[k] = pad_id;
                }
            }
        }
        OUT *o = ids + b * t_out + col0;
        if (ALIGNED) {
            const int4v vv = {v[0], v[1], v[2], v[3]};
            __builtin_nontemporal_store(make_quad<OUT>(vv), reinterpret_cast<typename Quad<OUT>::type *>(o));
            if (HAS_MASK)
                __builtin_nontemporal_store(m, reinterpret_cast<uint32_t *>(mask + b * t_out + col0));
        } else {
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                if (col0 + k < t_out) {
                    o[k] = (OUT)v[k];
                    if (HAS_MASK) mask[b * t_out + col0 + k] = (uint8_t)((m >> (8 * k)) & 1u);
                }
            }
        }
    }
}

static int grid_for(int64_t n_tiles)
{
    // enough workgroups to fill 256 CUs several times over; tiles beyond that are grid-strided
    const int64_t cap = 256 * 32;
    return (int)(n_tiles < cap ? (n_tiles > 0 ? n_tiles : 1) : cap);
}

}  // namespace dnatok

using namespace dnatok;

extern "C" int dnatok_char_table_create(const int32_t *lut_h, const int32_t *start_lut_h,
                                        int32_t pad_id, dnatok_char_t **out)
{
    DNATOK_REQUIRE(lut_h && out, DNATOK_E_INVALID, "dnatok_char_table_create: null argument");
    CharTableDev h;
    memcpy(h.lut, lut_h, sizeof(h.lut));
    memcpy(h.start, start_lut_h ? start_lut_h : lut_h, sizeof(h.start));
    dnatok_char_table *t = new dnatok_char_table();
    t->pad_id = pad_id;
    t->has_start = start_lut_h != nullptr;
    t->dev = nullptr;
    hipError_t e = hipMalloc((void **)&t->dev, sizeof(CharTableDev));
    if (e == hipSuccess) e = hipMemcpy(t->dev, &h, sizeof(h), hipMemcpyHostToDevice);
    if (e != hipSuccess) {
        set_error("dnatok_char_table_create: %s", hipGetErrorString(e));
        if (t->dev) (void)hipFree(t->dev);
        delete t;
        return DNATOK_E_HIP;
    }
    *out = t;
    return DNATOK_OK;
}

extern "C" void dnatok_char_table_destroy(dnatok_char_t *t)
{
    if (!t) return;
    if (t->dev) (void)hipFree(t->dev);
    delete t;
}

extern "C" int dnatok_char_encode_packed(const dnatok_char_t *t, const uint8_t *bytes, int64_t total,
                                         int64_t row_len, int32_t *ids, uint8_t *mask, void *stream)
{
    DNATOK_REQUIRE(t, DNATOK_E_INVALID, "dnatok_char_encode_packed: null argument");
    DNATOK_REQUIRE(total >= 0 && row_len >= 0, DNATOK_E_INVALID,
                   "dnatok_char_encode_packed: negative size");
    if (total == 0) return DNATOK_OK;
    DNATOK_REQUIRE(bytes && ids, DNATOK_E_INVALID, "dnatok_char_encode_packed: null buffer");
    DNATOK_REQUIRE(((uintptr_t)bytes & 3) == 0 && ((uintptr_t)ids & 15) == 0 &&
                       ((uintptr_t)mask & 3) == 0,
                   DNATOK_E_INVALID,
                   "dnatok_char_encode_packed: bytes/mask must be 4-byte and ids 16-byte aligned");
    hipStream_t s = (hipStream_t)stream;
    const int64_t n_tiles = (total + kCharTile - 1) / kCharTile;
    const int grid = grid_for(n_tiles);
    const bool use_start = t->has_start && row_len > 0;
    if (mask) {
        if (use_start)
            char_packed_kernel<true, true><<<grid, kCharThreads, 0, s>>>(bytes, total, row_len, t->dev, ids, mask);
        else
            char_packed_kernel<true, false><<<grid, kCharThreads, 0, s>>>(bytes, total, 1, t->dev, ids, mask);
    } else {
        if (use_start)
            char_packed_kernel<false, true><<<grid, kCharThreads, 0, s>>>(bytes, total, row_len, t->dev, ids, mask);
        else
            char_packed_kernel<false, false><<<grid, kCharThreads, 0, s>>>(bytes, total, 1, t->dev, ids, mask);
    }
    DNATOK_HIP_TRY(hipGetLastError());
    return DNATOK_OK;
}

namespace dnatok {

// Fused byte -> id -> embedding row: out[i, :] = emb[table[bytes[i]], :] without the id tensor in
// between.  A wave reads 64 bytes with one load, then copies the 64 rows one after the other,
// 16 bytes per lane and instruction (the row pointer is wave-uniform, so a copy instruction covers
// 1 KiB of the source row and 1 KiB of the output).  Write-bound: row_bytes per base.
constexpr int64_t kEmbedLdsBytes = 48 * 1024;      // embedding tables up to this size are staged in LDS

template <bool HAS_START, bool IN_LDS>
__global__ __launch_bounds__(kCharThreads) void char_embed_kernel(
    const uint8_t *__restrict__ bytes, int64_t total, int64_t row_len,
    const CharTableDev *__restrict__ tab, const uint8_t *__restrict__ emb, int32_t n_vocab,
    int64_t row_bytes, uint8_t *__restrict__ out)
{
    __shared__ int32_t lut[256];
    __shared__ int32_t start[256];
    extern __shared__ __align__(16) uint8_t s_emb[];          // the whole table when IN_LDS
    lut[threadIdx.x] = tab->lut[threadIdx.x];
    if (HAS_START) start[threadIdx.x] = tab->start[threadIdx.x];
    if (IN_LDS)
        for (int64_t o = (int64_t)threadIdx.x * 16; o < n_vocab * row_bytes; o += kCharThreads * 16)
            *reinterpret_cast<int4v *>(s_emb + o) = *reinterpret_cast<const int4v *>(emb + o);
    __syncthreads();

    const int lane = threadIdx.x & 63;
    const int64_t wave = (int64_t)blockIdx.x * (kCharThreads / 64) + (threadIdx.x >> 6);
    const int64_t n_waves = (int64_t)gridDim.x * (kCharThreads / 64);
    for (int64_t base = wave * 64; base < total; base += n_waves * 64) {
        const int64_t i = base + lane;
        int32_t id = -1;
        if (i < total) {
            const uint8_t c = bytes[i];
            id = (HAS_START && i % row_len == 0) ? start[c] : lut[c];
            if (id < 0 || id >= n_vocab) id = -1;                     // no such row: zeros
        }
        const int n_here = total - base < 64 ? (int)(total - base) : 64;
        // four rows per pass, so that four loads are in flight before the first store
        for (int b0 = 0; b0 < n_here; b0 += 4) {
            for (int64_t o = (int64_t)lane * 16; o < row_bytes; o += 64 * 16) {
                int4v v[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int32_t rid = __builtin_amdgcn_readlane(id, (b0 + j) & 63);
                    v[j] = int4v{0, 0, 0, 0};
                    if (rid >= 0) {
                        const int64_t at = (int64_t)rid * row_bytes + o;
                        v[j] = IN_LDS ? *reinterpret_cast<const int4v *>(s_emb + at)
                                      : *reinterpret_cast<const int4v *>(emb + at);
                    }
                }
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    if (b0 + j < n_here)
                        __builtin_nontemporal_store(v[j], reinterpret_cast<int4v *>(out + (base + b0 + j) * row_bytes + o));
            }
        }
    }
}

}  // namespace dnatok

extern "C" int dnatok_char_embed_packed(const dnatok_char_t *t, const uint8_t *bytes, int64_t total,
                                        int64_t row_len, const void *emb, int32_t n_vocab,
                                        int64_t row_bytes, void *out, void *stream)
{
    DNATOK_REQUIRE(t, DNATOK_E_INVALID, "dnatok_char_embed_packed: null argument");
    DNATOK_REQUIRE(total >= 0 && row_len >= 0 && n_vocab > 0 && row_bytes > 0, DNATOK_E_INVALID,
                   "dnatok_char_embed_packed: bad size");
    if (total == 0) return DNATOK_OK;
    DNATOK_REQUIRE(bytes && emb && out, DNATOK_E_INVALID, "dnatok_char_embed_packed: null buffer");
    DNATOK_REQUIRE(((uintptr_t)emb & 15) == 0 && ((uintptr_t)out & 15) == 0 && (row_bytes & 15) == 0,
                   DNATOK_E_INVALID,
                   "dnatok_char_embed_packed: embedding rows and output must be 16-byte aligned "
                   "(row_bytes a multiple of 16)");
    hipStream_t s = (hipStream_t)stream;
    const int grid = grid_for((total + 255) / 256);
    const bool use_start = t->has_start && row_len > 0;
    const int64_t table_bytes = (int64_t)n_vocab * row_bytes;
    const bool in_lds = table_bytes <= kEmbedLdsBytes;
    const size_t lds = in_lds ? (size_t)table_bytes : 0;
#define LAUNCH(S, L)                                                                              \
    char_embed_kernel<S, L><<<grid, kCharThreads, lds, s>>>(bytes, total, use_start ? row_len : 1, t->dev, \
                                                            (const uint8_t *)emb, n_vocab, row_bytes, (uint8_t *)out)
    if (use_start) { if (in_lds) LAUNCH(true, true); else LAUNCH(true, false); }
    else           { if (in_lds) LAUNCH(false, true); else LAUNCH(false, false); }
#undef LAUNCH
    DNATOK_HIP_TRY(hipGetLastError());
    return DNATOK_OK;
}

namespace dnatok {

// 2-bit packed bases (4 per byte, first base in the low bits, codes A C G T = 0 1 2 3) -> ids.
// HBM-bound and write-dominated: 0.25 byte read and sizeof(OUT) bytes written per base.  The
// workgroup first builds, in LDS, the four ids of every one of the 256 possible packed bytes;
// a lane then reads one packed byte (a wave covers 64 contiguous bytes), looks its four ids up
// with one LDS read and stores them contiguously (a wave covers 1 KiB of int32 ids).  Giving a
// lane four packed bytes and 64 contiguous output bytes instead measures 7 x slower: the four
// stores of a wave then each touch 64 lines.
constexpr int kUnpackSteps = 8;                                  // packed bytes per lane per tile
constexpr int kUnpackTile = kCharThreads * kUnpackSteps;         // 2048 packed bytes = 8192 bases

// QUADS: row_len % 4 == 0 and ids aligned to 4 elements, so the packed stream and the output are
// both flat and every packed byte owns one aligned group of four cells.  Otherwise rows are
// ceil(row_len / 4) packed bytes each and cells are stored one by one.
template <typename OUT, bool HAS_START, bool QUADS>
__global__ __launch_bounds__(kCharThreads) void char_unpack2bit_kernel(
    const uint8_t *__restrict__ packed, int64_t n_rows, int64_t row_len, int64_t row_packed,
    const CharTableDev *__restrict__ tab, OUT *__restrict__ ids)
{
    __shared__ int4v quad[256];
    __shared__ int32_t first[4];
    {
        const int32_t a = tab->lut['A'], c = tab->lut['C'], g = tab->lut['G'], t = tab->lut['T'];
        auto pick = [&](uint32_t code) { return code == 0 ? a : code == 1 ? c : code == 2 ? g : t; };
        const uint32_t b = threadIdx.x;
        quad[b] = int4v{pick(b & 3u), pick((b >> 2) & 3u), pick((b >> 4) & 3u), pick(b >> 6)};
        if (HAS_START && b < 4) first[b] = tab->start[(int)"ACGT"[b]];
    }
    __syncthreads();

    const int64_t n_packed = n_rows * row_packed;
    const int64_t n_tiles = (n_packed + kUnpackTile - 1) / kUnpackTile;
    for (int64_t tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
        const int64_t p0 = tile * kUnpackTile + threadIdx.x;
        uint8_t w[kUnpackSteps];
#pragma unroll
        for (int s = 0; s < kUnpackSteps; ++s) {
            const int64_t p = p0 + s * kCharThreads;
            w[s] = p < n_packed ? __builtin_nontemporal_load(packed + p) : (uint8_t)0;
        }
#pragma unroll
        for (int s = 0; s < kUnpackSteps; ++s) {
            const int64_t p = p0 + s * kCharThreads;
            if (p >= n_packed) continue;
            int4v v = quad[w[s]];
            if (QUADS) {
                if (HAS_START && (p * 4) % row_len == 0) v.x = first[w[s] & 3u];
                __builtin_nontemporal_store(make_quad<OUT>(v),
                                            reinterpret_cast<typename Quad<OUT>::type *>(ids + p * 4));
            } else {
                const int64_t b = p / row_packed;
                const int64_t col = (p - b * row_packed) * 4;
                if (HAS_START && col == 0) v.x = first[w[s] & 3u];
                OUT *o = ids + b * row_len + col;
                const int32_t vs[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                for (int k = 0; k < 4; ++k)
                    if (col + k < row_len) o[k] = (OUT)vs[k];
            }
        }
    }
}

template <typename OUT>
static int launch_unpack2bit(const dnatok_char_table *t, const uint8_t *packed, int64_t n_rows,
                             int64_t row_len, void *ids, hipStream_t s)
{
    const int64_t row_packed = (row_len + 3) / 4;
    const int64_t n_tiles = (n_rows * row_packed + kUnpackTile - 1) / kUnpackTile;
    const int grid = grid_for(n_tiles);
    const bool quads = row_len % 4 == 0 && ((uintptr_t)ids % (4 * sizeof(OUT))) == 0;
#define LAUNCH(S, Q)                                                                             \
    char_unpack2bit_kernel<OUT, S, Q><<<grid, kCharThreads, 0, s>>>(packed, n_rows, row_len,      \
                                                                     row_packed, t->dev, (OUT *)ids)
    if (t->has_start) { if (quads) LAUNCH(true, true); else LAUNCH(true, false); }
    else              { if (quads) LAUNCH(false, true); else LAUNCH(false, false); }
#undef LAUNCH
    DNATOK_HIP_TRY(hipGetLastError());
    return DNATOK_OK;
}

}  // namespace dnatok

extern "C" int dnatok_char_unpack_2bit(const dnatok_char_t *t, const uint8_t *packed, int64_t n_rows,
                                       int64_t row_len, void *ids, int32_t id_bytes, void *stream)
{
    DNATOK_REQUIRE(t, DNATOK_E_INVALID, "dnatok_char_unpack_2bit: null argument");
    DNATOK_REQUIRE(n_rows >= 0 && row_len >= 0, DNATOK_E_INVALID, "dnatok_char_unpack_2bit: negative size");
    DNATOK_REQUIRE(id_bytes == 1 || id_bytes == 4 || id_bytes == 8, DNATOK_E_INVALID,
                   "dnatok_char_unpack_2bit: id_bytes must be 1, 4 or 8 (got %d)", (int)id_bytes);
    if (n_rows == 0 || row_len == 0) return DNATOK_OK;
    DNATOK_REQUIRE(packed && ids, DNATOK_E_INVALID, "dnatok_char_unpack_2bit: null buffer");
    DNATOK_REQUIRE(((uintptr_t)ids % (size_t)id_bytes) == 0, DNATOK_E_INVALID,
                   "dnatok_char_unpack_2bit: ids not aligned to its element size");
    hipStream_t s = (hipStream_t)stream;
    if (id_bytes == 1) return launch_unpack2bit<uint8_t>(t, packed, n_rows, row_len, ids, s);
    if (id_bytes == 4) return launch_unpack2bit<int32_t>(t, packed, n_rows, row_len, ids, s);
    return launch_unpack2bit<int64_t>(t, packed, n_rows, row_len, ids, s);
}

namespace dnatok {

template <typename OUT>
static int launch_char_padded(const dnatok_char_table *t, const uint8_t *bytes, const int64_t *offsets,
                              int64_t n_rows, int64_t t_out, int pad_left, void *ids_v, uint8_t *mask,
                              hipStream_t s)
{
    OUT *ids = (OUT *)ids_v;
    const int64_t tiles_per_row = (t_out + kCharThreads * 4 - 1) / (kCharThreads * 4);
    const int grid = grid_for(n_rows * tiles_per_row);
    const bool aligned = (t_out % 4 == 0) && ((uintptr_t)ids % (4 * sizeof(OUT))) == 0 && ((uintptr_t)mask & 3) == 0;
    const bool hs = t->has_start;
#define LAUNCH(M, S, A)                                                                               \
    char_padded_kernel<OUT, M, S, A><<<grid, kCharThreads, 0, s>>>(bytes, offsets, n_rows, t_out,      \
                                                                   tiles_per_row, pad_left, t->pad_id, \
                                                                   t->dev, ids, mask)
    if (mask) {
        if (hs) { if (aligned) LAUNCH(true, true, true); else LAUNCH(true, true, false); }
        else    { if (aligned) LAUNCH(true, false, true); else LAUNCH(true, false, false); }
    } else {
        if (hs) { if (aligned) LAUNCH(false, true, true); else LAUNCH(false, true, false); }
        else    { if (aligned) LAUNCH(false, false, true); else LAUNCH(false, false, false); }
    }
#undef LAUNCH
    DNATOK_HIP_TRY(hipGetLastError());
    return DNATOK_OK;
}

}  // namespace dnatok

extern "C" int dnatok_char_encode_padded_as(const dnatok_char_t *t, const uint8_t *bytes,
                                            const int64_t *offsets, int64_t n_rows, int64_t t_out,
                                            int pad_left, void *ids, int32_t id_bytes, uint8_t *mask,
                                            void *stream)
{
    DNATOK_REQUIRE(t && offsets, DNATOK_E_INVALID, "dnatok_char_encode_padded: null argument");
    DNATOK_REQUIRE(n_rows >= 0 && t_out >= 0, DNATOK_E_INVALID,
                   "dnatok_char_encode_padded: negative size");
    DNATOK_REQUIRE(id_bytes == 1 || id_bytes == 2 || id_bytes == 4 || id_bytes == 8, DNATOK_E_INVALID,
                   "dnatok_char_encode_padded: id_bytes must be 1, 2, 4 or 8 (got %d)", (int)id_bytes);
    if (n_rows == 0 || t_out == 0) return DNATOK_OK;
    DNATOK_REQUIRE(ids, DNATOK_E_INVALID, "dnatok_char_encode_padded: null output");
    DNATOK_REQUIRE(((uintptr_t)ids % (size_t)id_bytes) == 0, DNATOK_E_INVALID,
                   "dnatok_char_encode_padded: ids not aligned to its element size");
    hipStream_t s = (hipStream_t)stream;
    switch (id_bytes) {
    case 1: return launch_char_padded<uint8_t>(t, bytes, offsets, n_rows, t_out, pad_left, ids, mask, s);
    case 2: return launch_char_padded<int16_t>(t, bytes, offsets, n_rows, t_out, pad_left, ids, mask, s);
    case 4: return launch_char_padded<int32_t>(t, bytes, offsets, n_rows, t_out, pad_left, ids, mask, s);
    default: return launch_char_padded<int64_t>(t, bytes, offsets, n_rows, t_out, pad_left, ids, mask, s);
    }
}

extern "C" int dnatok_char_encode_padded(const dnatok_char_t *t, const uint8_t *bytes,
                                         const int64_t *offsets, int64_t n_rows, int64_t t_out,
                                         int pad_left, int32_t *ids, uint8_t *mask, void *stream)
{
    return dnatok_char_encode_padded_as(t, bytes, offsets, n_rows, t_out, pad_left, ids, 4, mask, stream);
}
