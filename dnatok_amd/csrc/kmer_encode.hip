// Non-overlapping k-mer encoder with per-window fallback, tail handling, padding and mask.
//
// Persistent workgroups stage the tables in LDS once; after that every wave works alone on
// rows dealt round-robin.  A wave walks its row in steps of 256 units (a unit is a k-base
// window, or one of the trailing len % k characters).  Each lane owns 4 consecutive units: it
// takes its 4k bytes (requested one step earlier through a buffer descriptor of the row),
// turns them into base-4 digits through the LDS digit table, and looks the window up in the
// LDS table of the 4^k N-free windows.
//
//   * Plain step (every lane holds 4 plain windows or lies past the row's end, and the row's
//     write position is on a 128-byte line): token positions are known without a scan; each
//     lane issues one 16-byte id store and one 4-byte mask store (a wave covers 1 KiB + 256 B
//     contiguous).
//   * Any other step (a window holding N or a byte outside the alphabet, a window without an
//     id, the ragged end of a row, or a write position that an earlier expansion moved off
//     the line grid): unit token counts are prefix-summed across the wave with a DPP scan,
//     the lanes drop their tokens into a per-wave LDS staging area at their scanned
//     positions, and the wave writes the staged run back out as 16-byte groups, whole
//     128-byte lines at a time.  The tokens past the last whole line stay in LDS for the
//     next step of the row.  A step that yields more tokens than the staging area holds is
//     staged in several passes.
//     When the table spells every non-plain window character by character (the usual
//     grid-aligned tokenizer), the spelled tokens come from an LDS table; otherwise from the
//     global 5^k entry table and its expansion lists.
//
// Traffic: 1 byte read per base, 5 bytes written per token.
#include "common.hpp"

#include <limits.h>
#include <string.h>
#include <atomic>
#include <mutex>
#include <stdlib.h>
#include <unordered_map>
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
    int32_t *lut4r;          // the same ids indexed the way kmer_rows_kernel<..., ARITH> forms a window's code
    int arith;               // the digit table is the plain one (A C G T -> 0 1 2 3, N -> 4, nothing else,
    uint32_t fold;           // or lower case as well: fold = 0xDFDFDFDF, else 0xFFFFFFFF): digits by arithmetic
    int2 *entry;             // [5^k]  {id, 0} | {-len, offset into flat} | {INT_MIN, 0} = nothing known
    int32_t *flat;           // expansion lists
    // Running maxima of pad-to-longest calls.  Every stream that encodes with this table gets a
    // slot of its own (calls on one stream are ordered, calls on different streams may overlap and
    // must not share one); a stream beyond the kMaxSlots-th is served without a slot, by a clearing
    // launch on the caller's max_len.  A slot is two 64-bit words: the running maximum, tagged in
    // its upper half with the slot's generation, and the generation itself, which the padding pass
    // of a call bumps when it is done with the maximum.  A maximum of a later call is therefore
    // larger than anything an earlier call left behind, and the slot never has to be cleared (a
    // launch saved per call; replays of a captured call stay exact).
    unsigned long long *max_slots;
    unsigned long long *max_trees;       // kTreeWords words per slot (see kmer_team_kernel)
    mutable std::mutex slot_lock;
    mutable std::unordered_map<void *, int> slot_of_stream;
    // Batches of up to this many rows are encoded by kmer_team_kernel (a workgroup per row); -1: as
    // many rows as workgroups of that kernel fit the chip at once.  (dnatok_kmer_table_set_team_rows)
    std::atomic<int> team_rows{-1};
};

constexpr int kMaxSlots = 64;
constexpr int kMaxSlotStride = 32;       // 64-bit words between two slots (one 256-byte line each)
// A call whose kernel reports the maximum itself (kmer_team_kernel, publish) gathers it up a tree
// of atomics (climb_max_tree): kTreeWords words per slot.
using dnatok::kTreeRows;
using dnatok::kTreeWords;

namespace dnatok {

struct KmerArgs {
    const int8_t *digit;
    const int32_t *single, *lut4, *lut4r;
    uint32_t fold;
    const int2 *entry;
    const int32_t *flat;
    int32_t pad_id, missing_id;
};

constexpr int kKmerThreads = 256;         // kmer_team_kernel: four waves share a row
// kmer_rows_kernel: eight waves, a row each, share one copy of the tables.  Measured on the 6-mer
// workload (one-launch step): 128 threads 181 us, 256 170.9, 384 183 (12 waves per CU), 512 168.6,
// 768 177 (12 waves), 1024 as 256; N-free input 141.3 -> 137.5 us with 512.
constexpr int kRowsThreads = 512;
constexpr int kUnitsPerLane = 4;
constexpr int kWaveUnits = 64 * kUnitsPerLane;          // units one wave handles per step
// Staging area of one wave: kStageCap tokens in scanned order (+ room to read the last group whole).
constexpr int kStageCap = 512;
constexpr int kStageWords = kStageCap + 8;
// A shifted run is written out in whole units of kFlushCells cells (one 128-byte line of ids;
// a multiple of 4 that divides kStageCap); the cells past the last whole unit wait in LDS for
// the next step of the row, so that no line of the output is written in two pieces.
constexpr int kFlushCells = 32;
constexpr uint32_t kFlushMask = kFlushCells - 1;

// LDS digit entries: 0..3 for A C G T; flags above every window code (4^8 = 1 << 16) for N and
// for a byte outside the alphabet, so that "window code < 4^k" means "k plain bases".
constexpr uint32_t kDigN = 1u << 16;
constexpr uint32_t kDigBad = 1u << 17;
// In a window code c = sum of digit_i << 2 (K - 1 - i) the flags of the digits do not meet (the
// digits' own two bits stay below bit 16 for K <= 8): N flags land on even bits from 16 up,
// foreign-byte flags on odd bits from 17 up.
constexpr uint32_t kCodeBadBits = 0xAAAA0000u;
// byte offset past the end of every row descriptor (its stores are dropped), and the cache
// policy bits of the buffer stores (streaming: the output is not read again by the kernel)
constexpr uint32_t kDropOffset = 0x80000000u;
constexpr int kStoreAux = 2;

// 4 ids at element alignment (the compiler may not assume more; the addresses the kernels
// form are 16-byte aligned wherever the row layout allows)
typedef int32_t int4v_a4 __attribute__((ext_vector_type(4), aligned(4)));
typedef int32_t int4v __attribute__((ext_vector_type(4)));
typedef uint32_t u32_a1 __attribute__((aligned(1)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

__global__ void kmer_init_kernel(int32_t *max_len) { *max_len = 0; }

// Where a pad-to-longest call keeps its running maximum: slot[0] = generation << 32 | maximum,
// slot[1] = generation.
struct MaxRef {
    unsigned long long *slot;
    unsigned long long *tree;      // kTreeWords words of the slot's stream, all zero between calls
};

// Where a launch puts its rows and which rows it takes.
struct RowPlace {
    // packed output: row b's cells are ids[row_at[b] .. row_at[b + 1]) (and the same cells of the
    // mask), no padding; null: row b's cells start at ids[b * t_cap]
    const int64_t *row_at;
    // 0: every row; 1: the rows of at most kGroupsMaxUnits units; 2: the other rows (a batch of
    // mostly short rows with some long ones is split between kmer_groups_kernel and kmer_rows_kernel)
    int32_t row_class;
    // the rows' lengths are all that is written (the first pass of a packed encode)
    int32_t count_only;
};
constexpr int kGroupsMaxUnits = 384;

// Stores the group of 4 cells [e, e + 4) of a row whose cells are addressed from the
// 16-byte-aligned pointer pair (outA, moutA); only cells inside [lo, hi) are written.
__device__ __forceinline__ void store_group(int32_t *outA, uint8_t *moutA, int e, int lo, int hi,
                                            const int32_t *v, uint32_t mbyte)
{
    if (e >= lo && e + 4 <= hi) {
        int4v_a4 x = {v[0], v[1], v[2], v[3]};
        __builtin_nontemporal_store(x, reinterpret_cast<int4v_a4 *>(outA + e));
        if (moutA) __builtin_nontemporal_store((u32_a1)(mbyte * 0x01010101u), reinterpret_cast<u32_a1 *>(moutA + e));
    } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            if (e + i >= lo && e + i < hi) {
                outA[e + i] = v[i];
                if (moutA) moutA[e + i] = (uint8_t)mbyte;
            }
        }
    }
}

// Cells [from, to) of a row get the pad id and mask 0; the whole wave takes part.
__device__ __forceinline__ void pad_cells(int32_t *outA, uint8_t *moutA, int mis, int from, int to,
                                          int32_t pad_id, int lane)
{
    const int lo = mis + from, hi = mis + to;
    const int32_t v[4] = {pad_id, pad_id, pad_id, pad_id};
    for (int e = (lo & ~3) + 4 * lane; e < hi; e += 4 * 64) store_group(outA, moutA, e, lo, hi, v, 0u);
}

// Orders the LDS traffic of the lanes of one wave (they run in lockstep; this only keeps the
// compiler from moving LDS accesses across the point).
__device__ __forceinline__ void wave_sync()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// ARITH: the digit table is the plain one (see dnatok_kmer_table_create), and the digits of a lane
// with four whole windows come from the bytes by arithmetic on four bytes at a time instead of a
// trip to the digit table in LDS per byte: bits 1 and 2 of the ASCII code tell A, C, T and G
// apart (0, 1, 2, 3); v_perm_b32 with those bits as selectors rebuilds the byte they stand for,
// and a byte that differs from it is not one of the four.  The window code holds character i in
// bits 2i, 2i + 1 (a.lut4r is indexed that way).
// PLACED: the launch honours `place` (packed output, a class of rows, counting only); without it the
// argument is ignored and the rows lie a stride apart, so that the kernel of the padded layout is
// compiled exactly as it would be without these modes (as run-time choices they cost it 2 %).
template <int K, bool LUT4_LDS, bool CHARS, bool HAS_MASK, bool ARITH, bool PLACED = false>
__global__ __launch_bounds__(kRowsThreads) void kmer_rows_kernel(
    KmerArgs a, const uint8_t *__restrict__ bytes, const int64_t *__restrict__ offsets,
    int64_t n_rows, int64_t t_cap, int64_t fill_to, int32_t *__restrict__ ids,
    uint8_t *__restrict__ mask, int32_t *__restrict__ lengths, int32_t *__restrict__ status,
    int32_t *__restrict__ max_len, MaxRef mref, int publish, RowPlace place)
{
    constexpr uint32_t POW4 = 1u << (2 * K);
    __shared__ uint32_t s_dig[256];
    __shared__ int32_t s_single[256];
    __shared__ int32_t s_lut4[LUT4_LDS ? POW4 : 1];
    __shared__ int32_t s_spell[256];     // token a byte is spelled with inside a non-plain window
    __shared__ __attribute__((aligned(16))) int32_t s_stage[kRowsThreads / 64][kStageWords];

    for (int i = threadIdx.x; i < 256; i += kRowsThreads) {
        const int d = a.digit[i];
        s_dig[i] = d < 0 ? kDigBad : (d >= 4 ? kDigN : (uint32_t)d);
        s_single[i] = a.single[i];
        // a byte outside the alphabet counts as N inside a window
        s_spell[i] = a.single[(int)"ACGTN"[d < 0 || d > 4 ? 4 : d]];
    }
    const int32_t *const g_lut4 = ARITH ? a.lut4r : a.lut4;
    if (LUT4_LDS)
        for (uint32_t i = threadIdx.x; i < POW4; i += kRowsThreads) s_lut4[i] = g_lut4[i];
    // a window's code from the digit table's entries, character i at a time
    auto with_digit = [](uint32_t c, uint32_t v, int i) -> uint32_t {
        if (!ARITH) return (c << 2) + v;
        return c | ((v & (kDigN | kDigBad)) ? (v & (kDigN | kDigBad)) : (((v ^ (v >> 1)) & 3u) << (2 * i)));
    };
    __syncthreads();          // from here on every wave runs alone (one more barrier at the very end, with `publish`)

    const int lane = threadIdx.x & 63;
    int32_t *const buf = s_stage[__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6))];
    const int cap_all = t_cap > INT_MAX - 16 ? INT_MAX - 16 : (int)t_cap;
    const int fill_all = fill_to > cap_all ? cap_all : (int)fill_to;
    int64_t wave_max = 0;
    const unsigned long long slot_gen = mref.slot ? mref.slot[1] : 0ull;
    const int wave_in_wg = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int64_t wave = (int64_t)blockIdx.x * (kRowsThreads / 64) + wave_in_wg;
    const int64_t n_waves = (int64_t)gridDim.x * (kRowsThreads / 64);

    // Which rows the wave takes: every n_waves-th row; of a batch that is split by row class, the
    // long rows of every n_waves-th block of 64 rows -- the lanes look at a row each, so that the
    // short rows, which are nearly all of such a batch, cost a wave one load per 64 of them.
    const bool long_rows_only = PLACED && place.row_class == 2;
    int64_t cursor = long_rows_only ? wave * 64 : wave;
    uint64_t pending = 0;                                // (long_rows_only) rows of the block at `cursor` still to do
    auto next_row = [&]() -> int64_t {
        if (!long_rows_only) {
            const int64_t r = cursor;
            cursor += n_waves;
            return r < n_rows ? r : -1;
        }
        while (pending == 0) {
            if (cursor >= n_rows) return -1;
            const int64_t r = cursor + lane;
            bool is_long = false;
            if (r < n_rows) {
                const int64_t l = offsets[r + 1] - offsets[r];
                is_long = l / K + l % K > kGroupsMaxUnits;
            }
            pending = __ballot(is_long);
            if (pending == 0) cursor += n_waves * 64;
        }
        const int at = __builtin_ctzll(pending);
        pending &= pending - 1;
        const int64_t r = cursor + at;
        if (pending == 0) cursor += n_waves * 64;
        return r;
    };
    for (int64_t row = next_row(); row >= 0; row = next_row()) {
        const int64_t row_start = offsets[row];
        // positions inside a row are 32-bit: a row is shorter than 2^31 bytes
        const int len = (int)(offsets[row + 1] - row_start);
        const int full = len / K;
        const int n_units = full + (len - full * K);
        const uint8_t *src = bytes + row_start;
        // the row's cells: a stride apart, or (packed) where the rows before it end
        const int64_t cell0 = PLACED && place.row_at ? place.row_at[row] : row * t_cap;
        const int cap = !PLACED ? cap_all
                                : place.count_only ? 0 : place.row_at ? (int)(place.row_at[row + 1] - cell0) : cap_all;
        const int fill = PLACED && place.row_at ? 0 : fill_all;
        int32_t *out = ids + cell0;
        // cells are addressed from the 16-byte boundary at or below the row's first cell
        const int mis = (int)((reinterpret_cast<uintptr_t>(out) >> 2) & 3);
        int32_t *outA = out - mis;
        uint8_t *moutA = HAS_MASK ? mask + cell0 - mis : nullptr;
        const int lo = mis, hi_cap = mis + cap;
        int running = 0;
        int32_t my_status = 0;

        // The row's bytes are read through a buffer descriptor: a read past the row's end
        // returns 0 (never a base) instead of faulting, so the bytes of the next step are
        // requested without a branch, one step ahead of their use.
        const __amdgpu_buffer_rsrc_t rsrc =
            __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t *>(src), (short)0, len, 0x00020000);
        auto fetch = [&](uint32_t (&dst)[K], int unit0) {
            const int off = (unit0 + lane * kUnitsPerLane) * K;       // 4 windows = 4K bytes, unaligned
            int i = 0;
#pragma unroll
            for (; i + 4 <= K; i += 4) {
                const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(rsrc, off + 4 * i, 0, 0);
                dst[i] = v.x; dst[i + 1] = v.y; dst[i + 2] = v.z; dst[i + 3] = v.w;
            }
            if (i + 2 <= K) {
                const u32x2 v = __builtin_amdgcn_raw_buffer_load_b64(rsrc, off + 4 * i, 0, 0);
                dst[i] = v.x; dst[i + 1] = v.y;
                i += 2;
            }
            if (i < K) dst[i] = __builtin_amdgcn_raw_buffer_load_b32(rsrc, off + 4 * i, 0, 0);
        };
        // Stores of whole 4-cell groups go through buffer descriptors of the row as well: a lane
        // that has nothing to store points past the descriptor's end and the hardware drops its
        // store.  Every kind of step therefore issues the same stores (ids, mask) with no branch
        // around them, and the wait for the bytes requested one step earlier (the counter is in
        // issue order) can leave them in flight.
        const int vec_cap = cap < 0x1FFFFFF0 ? cap : 0x1FFFFFF0;      // cells a descriptor reaches
        const __amdgpu_buffer_rsrc_t rs_ids =
            __builtin_amdgcn_make_buffer_rsrc(out, (short)0, vec_cap * 4, 0x00020000);
        const __amdgpu_buffer_rsrc_t rs_msk = __builtin_amdgcn_make_buffer_rsrc(
            HAS_MASK ? mask + cell0 : reinterpret_cast<uint8_t *>(out), (short)0, HAS_MASK ? vec_cap : 0,
            0x00020000);
        // group of 4 cells starting at row cell r (whole = inside the row and the descriptor)
        auto store_vec = [&](bool whole, int r, const int32_t *v) {
            const int voff = whole ? r * 4 : (int)kDropOffset;
            const u32x4 x = {(uint32_t)v[0], (uint32_t)v[1], (uint32_t)v[2], (uint32_t)v[3]};
            __builtin_amdgcn_raw_buffer_store_b128(x, rs_ids, voff, 0, kStoreAux);
            if (HAS_MASK)
                __builtin_amdgcn_raw_buffer_store_b32(0x01010101u, rs_msk, whole ? r : (int)kDropOffset, 0, kStoreAux);
        };

        uint32_t w[K], wn[K];
        uint32_t code[kUnitsPerLane];
        int32_t t[kUnitsPerLane] = {0, 0, 0, 0};
        // digit of byte bi of this lane (LDS lookup)
        auto digit_of = [&](int bi) -> uint32_t { return s_dig[(w[bi >> 2] >> (8 * (bi & 3))) & 255u]; };

        // Waits for the bytes requested last.  Every way through a step that issues more memory
        // operations than the stores of store_vec starts with this: the compiler then knows the
        // request has landed on those ways, and on the remaining ones it can count the stores
        // between the request and its use exactly, and leave them in flight at the wait.
        auto settle = [&]() {
#pragma unroll
            for (int i = 0; i < K; ++i) asm volatile("" ::"v"(wn[i]));
        };
        fetch(wn, 0);
        settle();
        for (int u0 = 0; u0 < n_units; u0 += kWaveUnits) {
            const int ub = u0 + lane * kUnitsPerLane;
            const bool lane_full = ub + kUnitsPerLane <= full;     // 4 whole windows
            const bool empty = ub >= n_units;
#pragma unroll
            for (int i = 0; i < K; ++i) w[i] = wn[i];
            fetch(wn, u0 + kWaveUnits);
            // (ARITH) bytes of the lane that are none of A C G T, as nonzero bytes: only meaningful
            // for a lane whose bytes all lie inside the row (past its end the loads return zeros)
            uint32_t odd[ARITH ? K : 1];
            uint32_t odd_any = 0;
            if (ARITH) {
                // the digits of four bytes at a time, packed to one byte per word, then the
                // windows cut from the string of 2-bit digits
                uint32_t c8[K];
#pragma unroll
                for (int i = 0; i < K; ++i) {
                    const uint32_t d = w[i] & 0x06060606u;                       // digit << 1 in every byte
                    // pool of the 8-byte permute: byte 0 'A', 2 'C', 4 'T', 6 'G'
                    odd[i] = (w[i] ^ __builtin_amdgcn_perm(0x00470054u, 0x00430041u, d)) & a.fold;
                    odd_any |= odd[i];
                    const uint32_t x1 = (d << 6) | d;                            // bits 7..10, 23..26: two digits each
                    const uint32_t x2 = (x1 << 12) | x1;                         // bits 19..26: the four digits
                    c8[i] = (x2 >> 19) & 255u;
                }
                uint32_t str[(K + 3) / 4 + 1];
#pragma unroll
                for (int q = 0; q < (K + 3) / 4 + 1; ++q) {
                    uint32_t v = 0;
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (4 * q + e < K) v |= c8[4 * q + e] << (8 * e);
                    str[q] = v;
                }
#pragma unroll
                for (int j = 0; j < kUnitsPerLane; ++j) {
                    constexpr uint32_t kCodeMask = POW4 - 1;
                    const int bit = 2 * K * j;
                    const uint64_t two = ((uint64_t)str[(bit >> 5) + 1] << 32) | str[bit >> 5];
                    code[j] = (uint32_t)(two >> (bit & 31)) & kCodeMask;
                }
            } else {
#pragma unroll
                for (int j = 0; j < kUnitsPerLane; ++j) {
                    uint32_t c = 0;
#pragma unroll
                    for (int i = 0; i < K; ++i) c = (c << 2) + digit_of(j * K + i);
                    code[j] = c;
                }
            }
#pragma unroll
            for (int j = 0; j < kUnitsPerLane; ++j) {
                const uint32_t idx = code[j] & (POW4 - 1);
                t[j] = LUT4_LDS ? s_lut4[idx] : g_lut4[idx];
            }
            const uint32_t any_flag = ARITH ? odd_any : (code[0] | code[1] | code[2] | code[3]);
            const bool fast = lane_full && (ARITH ? any_flag == 0 : any_flag < POW4) && (t[0] | t[1] | t[2] | t[3]) >= 0;
            const uint64_t rest_mask = __ballot(!fast && !empty);
            const int A = mis + running;           // cell the step's first token goes to

            // Tokens per unit and per lane, and their prefix sum over the wave.  Done for every
            // step, also the plain ones that know their positions without it: the step's token
            // count is then a scalar defined on one path only.  (A scalar that only one side of
            // a branch defines is given a filler definition read from an arbitrary vector
            // register; when that register is one the next step's bytes are being loaded into,
            // the filler waits for the load.)
            // per unit: cnt = number of tokens; ex/ey = entry of a window that is not plain
            int32_t cnt[kUnitsPerLane], ex[kUnitsPerLane], ey[kUnitsPerLane];
            uint32_t lane_cnt = 0;
            if (fast) {
                lane_cnt = kUnitsPerLane;
            } else if (lane_full) {
                if (ARITH && odd_any) {
                    // which windows hold a byte that is none of the four (kDigN on their code), and
                    // whether such a byte is no N either (kDigBad): the byte that bits 1..3 of a
                    // byte stand for, with N in the pool
                    uint32_t foreign = 0;
#pragma unroll
                    for (int i = 0; i < K; ++i) {
                        const uint32_t sel = (w[i] >> 1) & 0x07070707u;           // A 0, C 1, T 2, G 3, N 7
                        foreign |= w[i] ^ __builtin_amdgcn_perm(0x4E000000u, 0x47544341u, sel);
                    }
                    foreign &= a.fold;
#pragma unroll
                    for (int j = 0; j < kUnitsPerLane; ++j) {
                        uint32_t hit = 0;
#pragma unroll
                        for (int i = 0; i < K; ++i) {
                            const int bi = j * K + i;
                            hit |= odd[bi >> 2] & (0xFFu << (8 * (bi & 3)));
                        }
                        if (hit) code[j] |= foreign ? (kDigN | kDigBad) : kDigN;
                    }
                }
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
                    // the foreign-byte flag of digit i sits at bit 17 + 2 (K - 1 - i) of the window's
                    // code, the N flag one below it: an odd bit above 16 is a foreign byte
                    if (code[j] & kCodeBadBits) my_status |= DNATOK_ROW_INVALID_BYTE;
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
                            c = with_digit(c, v, i);
                            if (v & kDigBad) my_status |= DNATOK_ROW_INVALID_BYTE;
                            c5 = c5 * 5 + ((v & (kDigN | kDigBad)) ? 4 : (int)v);
                        }
                        int32_t id = -1;
                        if (c < POW4) id = LUT4_LDS ? s_lut4[c] : g_lut4[c];
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
            if (PLACED && place.count_only) {      // (the step's tokens are counted, not made)
                running += (int)step_total;
                continue;
            }

            // what the step's common store (one 4-cell group per lane) will write
            bool sv_whole = false;
            int sv_r = 0;
            int32_t sv_v[4] = {0, 0, 0, 0};

            if (rest_mask == 0 && (A & (int)kFlushMask) == 0) {
                // every lane is plain or past the end, and the run starts on a 16-byte boundary:
                // positions are known without a scan
                const int r = running + lane * kUnitsPerLane;
                sv_whole = fast && r + 4 <= vec_cap;
                sv_r = r;
#pragma unroll
                for (int j = 0; j < kUnitsPerLane; ++j) sv_v[j] = t[j];
                if (__ballot(fast && !sv_whole)) {                 // row cut at t_cap
                    settle();
                    if (fast && !sv_whole) store_group(outA, moutA, mis + r, lo, hi_cap, t, 1u);
                }
            } else {
            // ---- staged step ----
            // staged index 0 is the cell at the last multiple of kFlushCells at or below A; the first
            // `carry` entries are the tokens the previous step left over (at the start of a row:
            // cells of the neighbouring row, never written)
            const uint32_t carry = (uint32_t)A & kFlushMask;
            const uint32_t n_avail = carry + step_total;
            const uint32_t s0 = carry + (inc - lane_cnt);
            const bool last_step = u0 + kWaveUnits >= n_units;
            const int A_end = A + (int)step_total;
            const int hi = last_step && A_end < hi_cap ? A_end : hi_cap;

            // the tokens of a lane's units one unit at a time, from the row's bytes in memory (the
            // ragged end of a row: whole windows first, then single characters); put(s, tok)
            auto emit_units = [&](auto put, uint32_t s) {
    #pragma unroll 1
                for (int j = 0; j < kUnitsPerLane; ++j) {
                    const int u = ub + j;
                    if (u < full) {
                        uint32_t c = 0;
                        int c5 = 0;
    #pragma unroll
                        for (int i = 0; i < K; ++i) {
                            const uint32_t v = s_dig[src[u * K + i]];
                            c = with_digit(c, v, i);
                            c5 = c5 * 5 + ((v & (kDigN | kDigBad)) ? 4 : (int)v);
                        }
                        int32_t id = -1;
                        if (c < POW4) id = LUT4_LDS ? s_lut4[c] : g_lut4[c];
                        if (id >= 0) {
                            put(s, id);
                            ++s;
                        } else {
                            const int2 e = a.entry[c5];
                            if (e.x >= 0 || e.x == INT_MIN) {
                                put(s, e.x >= 0 ? e.x : a.missing_id);
                                ++s;
                            } else {
                                for (int q = 0; q < -e.x; ++q) put(s + q, a.flat[e.y + q]);
                                s += -e.x;
                            }
                        }
                    } else if (u < n_units) {
                        put(s, s_single[src[full * K + (u - full)]]);
                        ++s;
                    }
                }
            };
            // the lanes' tokens in scanned order; put(s, tok) places token s of the staged run
            auto produce = [&](auto put) {
                uint32_t s = s0;
                if (fast) {
    #pragma unroll
                    for (int j = 0; j < kUnitsPerLane; ++j) put(s + j, t[j]);
                } else if (lane_full) {
                    // The tokens the lane's bytes are spelled with: all lookups on their way together
                    // (a window at a time they are four trips to LDS in a row, on the step that
                    // takes longest anyway), where the registers allow it (k <= 6: more would
                    // cost the kernel a wave per SIMD).
                    constexpr bool kSpellAhead = CHARS && K <= 6;
                    int32_t sp[kSpellAhead ? kUnitsPerLane * K : 1];
                    if (kSpellAhead) {
    #pragma unroll
                        for (int bi = 0; bi < kUnitsPerLane * K; ++bi)
                            sp[bi] = s_spell[(w[bi >> 2] >> (8 * (bi & 3))) & 255u];
                    }
    #pragma unroll
                    for (int j = 0; j < kUnitsPerLane; ++j) {
                        if (code[j] < POW4 && t[j] >= 0) {
                            put(s, t[j]);
                            ++s;
                        } else if (CHARS) {
    #pragma unroll
                            for (int i = 0; i < K; ++i) {
                                const int bi = j * K + i;
                                put(s + i, kSpellAhead ? sp[kSpellAhead ? bi : 0] : s_spell[(w[bi >> 2] >> (8 * (bi & 3))) & 255u]);
                            }
                            s += K;
                        } else if (ex[j] >= 0) {
                            put(s, ex[j]);
                            ++s;
                        } else if (ex[j] == INT_MIN) {
                            put(s, a.missing_id);
                            ++s;
                        } else {
                            for (int e = 0; e < -ex[j]; ++e) put(s + e, a.flat[ey[j] + e]);
                            s += -ex[j];
                        }
                    }
                } else if (!empty) {
                    emit_units(put, s);
                }
            };
            auto group_at = [&](uint32_t g, int32_t *v) {
                const int4v x = *reinterpret_cast<const int4v *>(buf + 4 * g);
                v[0] = x.x; v[1] = x.y; v[2] = x.z; v[3] = x.w;
            };

            // How a step with more tokens than the staging area holds is written out.  In passes
            // for k <= 6: that kernel has 123 registers either way (4 waves per SIMD), and measured
            // 1-3 % faster on the 6-mer workload than the same kernel with 78 registers and the
            // cell-by-cell form (at 4 and at 5 waves per SIMD).  Cell by cell for k = 7, 8, where
            // the passes push the kernel beyond 128 registers (3 waves per SIMD).
            constexpr bool kStageInPasses = K <= 6;
            if (n_avail <= (uint32_t)kStageCap) {
                produce([&](uint32_t s, int32_t tok) { buf[s] = tok; });
                wave_sync();
                // whole groups; the row's last step also writes the group it leaves unfilled
                const uint32_t n_groups = last_step ? (n_avail + 3) >> 2 : (n_avail & ~kFlushMask) >> 2;
                const int e0 = A & ~(int)kFlushMask;
                {
                    // groups 0..63: one per lane, left to the step's common store
                    const int e = e0 + 4 * lane;
                    const bool mine = (uint32_t)lane < n_groups;
                    group_at(lane, sv_v);
                    sv_whole = mine && e >= lo && e + 4 <= hi && e - mis + 4 <= vec_cap;
                    sv_r = e - mis;
                    if (__ballot(mine && !sv_whole)) {             // row's first or last cells
                        settle();
                        if (mine && !sv_whole) store_group(outA, moutA, e, lo, hi, sv_v, 1u);
                    }
                }
                if (n_groups > 64) {
                    settle();
                    for (uint32_t g = lane + 64; g < n_groups; g += 64) {
                        int32_t v[4];
                        group_at(g, v);
                        store_group(outA, moutA, e0 + 4 * (int)g, lo, hi, v, 1u);
                    }
                }
                const uint32_t left = last_step ? 0u : (n_avail & kFlushMask);
                int32_t keep = 0;
                if ((uint32_t)lane < left) keep = buf[(n_avail & ~kFlushMask) + lane];
                wave_sync();
                if ((uint32_t)lane < left) buf[lane] = keep;
            } else if (kStageInPasses) {
                // more than kStageCap tokens in one step: staged and written out in several passes
                settle();
                for (uint32_t pass = 0; pass < n_avail; pass += kStageCap) {
                    produce([&](uint32_t s, int32_t tok) {
                        const uint32_t rel = s - pass;
                        if (rel < (uint32_t)kStageCap) buf[rel] = tok;
                    });
                    wave_sync();
                    const bool final_pass = pass + kStageCap >= n_avail;
                    const uint32_t count = final_pass ? n_avail - pass : (uint32_t)kStageCap;
                    const uint32_t n_groups = final_pass && last_step ? (count + 3) >> 2 : (count & ~kFlushMask) >> 2;
                    const int e0 = (A & ~(int)kFlushMask) + (int)pass;
                    for (uint32_t g = lane; g < n_groups; g += 64) {
                        int32_t v[4];
                        group_at(g, v);
                        store_group(outA, moutA, e0 + 4 * (int)g, lo, hi, v, 1u);
                    }
                    const uint32_t left = final_pass && !last_step ? (count & kFlushMask) : 0u;
                    int32_t keep = 0;
                    if ((uint32_t)lane < left) keep = buf[(count & ~kFlushMask) + lane];
                    wave_sync();
                    if ((uint32_t)lane < left) buf[lane] = keep;
                    wave_sync();
                }
            } else {
                // More than kStageCap tokens in one step, k >= 7: every lane writes its own tokens
                // cell by cell, reading the row's bytes from memory as the lanes of a ragged end
                // do.  Rare and slow on purpose: the passes above keep everything a step computes
                // alive across a loop, which for these k costs the kernel a wave per SIMD.  The
                // tokens past the last whole unit also go to the staging area, where the next
                // step looks for them.
                settle();
                const int e0 = A & ~(int)kFlushMask;
                const uint32_t keep_from = last_step ? 0xFFFFFFFFu : (n_avail & ~kFlushMask);
                int32_t left_over = 0;
                if ((uint32_t)lane < carry) left_over = buf[lane];
                wave_sync();
                auto put_cell = [&](uint32_t s, int32_t tok) {
                    const int e = e0 + (int)s;
                    if (e >= lo && e < hi) {
                        outA[e] = tok;
                        if (HAS_MASK) moutA[e] = 1;
                    }
                    if (s >= keep_from) buf[s - keep_from] = tok;
                };
                if ((uint32_t)lane < carry) put_cell((uint32_t)lane, left_over);
                if (!empty) emit_units(put_cell, s0);
                wave_sync();
            }
            }
            store_vec(sv_whole, sv_r, sv_v);
            running += (int)step_total;
        }

        const int stored = running < cap ? running : cap;
        int32_t st = 0;
        if (__ballot(my_status & DNATOK_ROW_INVALID_BYTE)) st |= DNATOK_ROW_INVALID_BYTE;
        if (__ballot(my_status & DNATOK_ROW_MISSING_KMER)) st |= DNATOK_ROW_MISSING_KMER;
        if (PLACED ? running > cap : running > t_cap) st |= DNATOK_ROW_TRUNCATED;
        if (lane == 0) {
            lengths[row] = (int32_t)running;
            if (status) status[row] = st;
        }
        if (stored > wave_max) wave_max = stored;
        if (fill > stored) pad_cells(outA, moutA, mis, stored, fill, a.pad_id, lane);
    }
    if (publish) {
        // no padding pass follows: the workgroups' maxima go up the tree (climb_max_tree)
        __shared__ uint32_t s_wave_max[kRowsThreads / 64];
        if (lane == 0) s_wave_max[wave_in_wg] = (uint32_t)wave_max;
        __syncthreads();
        if (threadIdx.x == 0) {
            uint32_t m = 0;
#pragma unroll
            for (int q = 0; q < kRowsThreads / 64; ++q) m = s_wave_max[q] > m ? s_wave_max[q] : m;
            const unsigned long long mine = (unsigned long long)m + 1;
            const unsigned long long before = atomicAdd(mref.tree + (blockIdx.x >> 2), mine << (16 * (blockIdx.x & 3)));
            climb_max_tree(mref.tree, blockIdx.x, gridDim.x, mine, before, max_len);
        }
        return;
    }
    // one atomic per wave at most, skipped when another wave already published a larger value
    if (mref.slot) {
        // (the first wave publishes even a maximum of 0: the slot then carries this call's tag)
        const unsigned long long v = (slot_gen << 32) | (unsigned long long)wave_max;
        if (lane == 0 && (wave_max > 0 || wave == 0) && __builtin_nontemporal_load(mref.slot) < v)
            atomicMax(mref.slot, v);
    } else if (max_len && lane == 0 && wave_max > 0 &&
               (int64_t)__builtin_nontemporal_load(max_len) < wave_max) {
        atomicMax(max_len, (int32_t)wave_max);
    }
}

// ---- short rows: sixteen lanes per row -----------------------------------------------------------
//
// A read of a few hundred bases is one step of kmer_rows_kernel in which a sixth of the lanes
// take part, and the row's fixed work is then all there is.  Here a row belongs to 16 lanes (four
// rows to a wave, sixteen to a workgroup) that walk it in steps of 64 windows: the digits by
// arithmetic on the bytes (the plain digit table only, see ARITH above), the positions by a scan
// over the 16 lanes (DPP row operations stay inside them), the tokens stored by the lanes
// themselves, a 16-byte store for a lane of four plain windows on a 16-byte boundary and single
// cells otherwise: no staging, no LDS beyond the tables.  For tables that spell every window
// without an id by its characters (CHARS above) and row strides of at most kGroupsMaxStride cells.
constexpr int kGroupThreads = 256;
constexpr int kGroupsMaxStride = 384;

// inclusive sum over the 16 lanes of a DPP row
__device__ __forceinline__ uint32_t row16_inclusive_sum(uint32_t v)
{
    v += dpp_row_shr_zero<1>(v);
    v += dpp_row_shr_zero<2>(v);
    v += dpp_row_shr_zero<4>(v);
    v += dpp_row_shr_zero<8>(v);
    return v;
}

// the value of the last of a lane's 16
__device__ __forceinline__ uint32_t row16_last(uint32_t v)
{
    const int src = (int)((threadIdx.x & 63) | 15);
    return (uint32_t)__builtin_amdgcn_ds_bpermute(src << 2, (int)v);
}

template <int K, bool LUT4_LDS, bool HAS_MASK>
__global__ __launch_bounds__(kGroupThreads) void kmer_groups_kernel(
    KmerArgs a, const uint8_t *__restrict__ bytes, const int64_t *__restrict__ offsets,
    int64_t n_rows, int64_t t_cap, int64_t fill_to, int32_t *__restrict__ ids,
    uint8_t *__restrict__ mask, int32_t *__restrict__ lengths, int32_t *__restrict__ status,
    int32_t *__restrict__ max_len, MaxRef mref, int publish, RowPlace place)
{
    constexpr uint32_t POW4 = 1u << (2 * K);
    constexpr int kLaneBytes = kUnitsPerLane * K;                 // bytes of a lane's four windows
    __shared__ int32_t s_single[256];
    __shared__ int32_t s_spell[256];
    __shared__ int32_t s_lut4[LUT4_LDS ? POW4 : 1];
    __shared__ uint32_t s_wave_max[kGroupThreads / 64];
    for (int i = threadIdx.x; i < 256; i += kGroupThreads) {
        const int d = a.digit[i];
        s_single[i] = a.single[i];
        s_spell[i] = a.single[(int)"ACGTN"[d < 0 || d > 4 ? 4 : d]];
    }
    if (LUT4_LDS)
        for (uint32_t i = threadIdx.x; i < POW4; i += kGroupThreads) s_lut4[i] = a.lut4r[i];
    __syncthreads();

    const int lane = threadIdx.x & 63, gl = lane & 15;
    const int cap_all = t_cap > INT_MAX - 16 ? INT_MAX - 16 : (int)t_cap;
    const int fill_all = fill_to > cap_all ? cap_all : (int)fill_to;
    const int64_t group = ((int64_t)blockIdx.x * kGroupThreads + threadIdx.x) >> 4;
    const int64_t n_groups = (int64_t)gridDim.x * (kGroupThreads / 16);
    const unsigned long long slot_gen = mref.slot ? mref.slot[1] : 0ull;
    const int64_t total = offsets[n_rows];
    uint32_t group_max = 0;

    // every group of the wave makes the same number of trips (a group without a row idles), so
    // that the wave's loads can share one descriptor per trip
    const int64_t wave_first = group - (lane >> 4);
    for (int64_t row0 = wave_first; row0 < n_rows; row0 += n_groups) {
        const int64_t row = row0 + (lane >> 4);
        bool have = row < n_rows;
        const int64_t start = have ? offsets[row] : 0;
        int len = have ? (int)(offsets[row + 1] - start) : 0;
        if (place.row_class == 1 && len / K + len % K > kGroupsMaxUnits) {     // (kmer_rows_kernel's row)
            have = false;
            len = 0;
        }
        const int full = len / K, tail = len - full * K;
        const int n_slots = full + (tail ? 1 : 0);                // windows, and one slot for the trailing characters
        // the row's cells: a stride apart, or (packed) where the rows before it end
        const int64_t cell0 = !have ? 0 : place.row_at ? place.row_at[row] : row * t_cap;
        const int cap = place.count_only || !have ? 0 : place.row_at ? (int)(place.row_at[row + 1] - cell0) : cap_all;
        const int fill = place.row_at || !have ? 0 : fill_all;
        int32_t *out = ids + cell0;
        uint8_t *mout = HAS_MASK ? mask + cell0 : nullptr;
        int running = 0;
        bool foreign_seen = false;

        const int steps = (n_slots + 63) >> 6;
        const int wave_steps = (int)wave_max_u32((uint32_t)steps);        // (wave-uniform loop: the loads are wave-wide)
        for (int st = 0; st < wave_steps; ++st) {
            const int wb = st * 64 + gl * kUnitsPerLane;          // the lane's first window
            // the lane's 4K bytes, a word at a time; what lies past the row's end (the next rows'
            // bytes) is read and ignored, what lies past the end of the batch is not read
            const int64_t pos = start + (int64_t)wb * K;
            uint32_t w[K];
#pragma unroll
            for (int i = 0; i < K; ++i) {
                const int64_t at = pos + 4 * i;
                uint32_t v = 0;
                if (wb < n_slots) {
                    if (at + 4 <= total) {
                        v = *reinterpret_cast<const u32_a1 *>(bytes + at);
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            if (at + e < total) v |= (uint32_t)bytes[at + e] << (8 * e);
                    }
                }
                w[i] = v;
            }
            // digits, codes and the bytes that are no base, as in kmer_rows_kernel<..., ARITH>
            uint32_t odd[K], c8[K];
#pragma unroll
            for (int i = 0; i < K; ++i) {
                const uint32_t d = w[i] & 0x06060606u;
                odd[i] = (w[i] ^ __builtin_amdgcn_perm(0x00470054u, 0x00430041u, d)) & a.fold;
                const uint32_t x1 = (d << 6) | d, x2 = (x1 << 12) | x1;
                c8[i] = (x2 >> 19) & 255u;
            }
            uint32_t str[(K + 3) / 4 + 1];
#pragma unroll
            for (int q = 0; q < (K + 3) / 4 + 1; ++q) {
                uint32_t v = 0;
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (4 * q + e < K) v |= c8[4 * q + e] << (8 * e);
                str[q] = v;
            }
            // per slot: its token count, and for a plain window its id
            int32_t t[kUnitsPerLane];
            uint32_t cnt[kUnitsPerLane], lane_cnt = 0;
            bool spelled_any = false;
#pragma unroll
            for (int j = 0; j < kUnitsPerLane; ++j) {
                const int bit = 2 * K * j;
                const uint64_t two = ((uint64_t)str[(bit >> 5) + 1] << 32) | str[bit >> 5];
                const uint32_t code = (uint32_t)(two >> (bit & 31)) & (POW4 - 1);
                t[j] = LUT4_LDS ? s_lut4[code] : a.lut4r[code];
                uint32_t hit = 0;
#pragma unroll
                for (int i = 0; i < K; ++i) {
                    const int bi = j * K + i;
                    hit |= odd[bi >> 2] & (0xFFu << (8 * (bi & 3)));
                }
                const int slot = wb + j;
                uint32_t c = 0;
                if (slot < full) {
                    c = (hit == 0 && t[j] >= 0) ? 1u : (uint32_t)K;
                    if (c != 1u) { t[j] = -1; spelled_any = true; }
                } else if (slot == full && tail) {
                    c = (uint32_t)tail;
                    t[j] = -2;                                     // the trailing characters
                }
                cnt[j] = c;
                lane_cnt += c;
            }
            // a byte of a window (not of the trailing characters) that is neither a base nor N: the
            // row is flagged
            if (spelled_any) {
                const int in_windows = full - wb < kUnitsPerLane ? (full - wb) * K : kLaneBytes;     // bytes of whole windows
                uint32_t f = 0;
#pragma unroll
                for (int i = 0; i < K; ++i) {
                    const uint32_t sel = (w[i] >> 1) & 0x07070707u;               // A 0, C 1, T 2, G 3, N 7
                    const int nb = in_windows - 4 * i;
                    const uint32_t m = nb >= 4 ? 0xFFFFFFFFu : (nb <= 0 ? 0u : ((1u << (8 * nb)) - 1u));
                    f |= (w[i] ^ __builtin_amdgcn_perm(0x4E000000u, 0x47544341u, sel)) & m;
                }
                if (f & a.fold) foreign_seen = true;
            }
            const uint32_t inc = row16_inclusive_sum(lane_cnt);
            const uint32_t step_total = row16_last(inc);
            uint32_t s = (uint32_t)running + inc - lane_cnt;      // cell of the lane's first token

            auto byte_of = [&](int bi) -> uint32_t { return (w[bi >> 2] >> (8 * (bi & 3))) & 255u; };
            if (lane_cnt == kUnitsPerLane && cnt[0] == 1 && cnt[1] == 1 && cnt[2] == 1 && cnt[3] == 1 &&
                (t[0] | t[1] | t[2] | t[3]) >= 0 && (int)s + 4 <= cap && ((reinterpret_cast<uintptr_t>(out + s) & 15) == 0)) {
                const int4v x = {t[0], t[1], t[2], t[3]};
                __builtin_nontemporal_store(x, reinterpret_cast<int4v *>(out + s));
            } else if (lane_cnt) {
#pragma unroll
                for (int j = 0; j < kUnitsPerLane; ++j) {
                    if (cnt[j] == 0) continue;
                    if (t[j] >= 0) {
                        if ((int)s < cap) out[s] = t[j];
                        s += 1;
                    } else if (t[j] == -1) {
#pragma unroll
                        for (int i = 0; i < K; ++i)
                            if ((int)s + i < cap) out[s + i] = s_spell[byte_of(j * K + i)];
                        s += K;
                    } else {
#pragma unroll
                        for (int i = 0; i < K - 1; ++i)
                            if (i < tail && (int)s + i < cap) out[s + i] = s_single[byte_of(j * K + i)];
                        s += (uint32_t)tail;
                    }
                }
            }
            running += (int)step_total;
        }

        // the row's end: mask, padding, length and status, by the row's 16 lanes
        const int stored = running < cap ? running : cap;
        const int upto = fill > stored ? fill : stored;
        if (HAS_MASK && have) {
            for (int c = 4 * gl; c < upto; c += 64) {
                const int ones = stored - c;                       // cells of this word that hold a token
                const uint32_t v = ones >= 4 ? 0x01010101u : (ones <= 0 ? 0u : (0x01010101u >> (8 * (4 - ones))));
                if (c + 4 <= upto && ((reinterpret_cast<uintptr_t>(mout) & 3) == 0)) {
                    *reinterpret_cast<uint32_t *>(mout + c) = v;
                } else {
                    for (int e = 0; e < 4; ++e)
                        if (c + e < upto) mout[c + e] = (uint8_t)((v >> (8 * e)) & 1u);
                }
            }
        }
        if (have) {
            for (int c = (stored & ~3) + 4 * gl; c < fill; c += 64) {
                if (c >= stored && c + 4 <= fill && ((reinterpret_cast<uintptr_t>(out) & 15) == 0)) {
                    const int4v x = {a.pad_id, a.pad_id, a.pad_id, a.pad_id};
                    __builtin_nontemporal_store(x, reinterpret_cast<int4v *>(out + c));
                } else {
                    for (int e = 0; e < 4; ++e)
                        if (c + e >= stored && c + e < fill) out[c + e] = a.pad_id;
                }
            }
        }
        const uint64_t bad = __ballot(foreign_seen);
        if (have && gl == 0) {
            lengths[row] = running;
            if (status) {
                int32_t v = ((bad >> (lane & 48)) & 0xFFFFull) ? DNATOK_ROW_INVALID_BYTE : 0;
                if (running > cap) v |= DNATOK_ROW_TRUNCATED;
                status[row] = v;
            }
        }
        if (have && (uint32_t)stored > group_max) group_max = (uint32_t)stored;
    }

    // the longest row: as kmer_rows_kernel reports it
    const uint32_t wmax = wave_max_u32(group_max);
    if (publish) {
        if (lane == 0) s_wave_max[threadIdx.x >> 6] = wmax;
        __syncthreads();
        if (threadIdx.x == 0) {
            uint32_t m = 0;
#pragma unroll
            for (int q = 0; q < kGroupThreads / 64; ++q) m = s_wave_max[q] > m ? s_wave_max[q] : m;
            publish_max(mref.tree, m, max_len);
        }
        return;
    }
    if (mref.slot) {
        const unsigned long long v = (slot_gen << 32) | (unsigned long long)wmax;
        const bool first_wave = blockIdx.x == 0 && threadIdx.x < 64;
        if (lane == 0 && (wmax > 0 || first_wave) && __builtin_nontemporal_load(mref.slot) < v) atomicMax(mref.slot, v);
    } else if (max_len && lane == 0 && wmax > 0 && (uint32_t)__builtin_nontemporal_load(max_len) < wmax) {
        atomicMax(max_len, (int32_t)wmax);
    }
}

// ---- few rows: a workgroup per row ---------------------------------------------------------------
//
// With fewer rows than workgroups fit the chip (one 256-row batch), a wave per row leaves most of
// the chip idle while every wave walks its row step by step.  Here the four waves of a workgroup
// share a row: wave w takes steps w, w + 4, ...; the token counts of the four steps of a round go
// through LDS, so that every wave knows where its tokens start.  A wave writes its run by itself,
// whole 16-byte groups and single cells at both ends (no waiting for whole lines as in
// kmer_rows_kernel: this kernel is for batches that are bound by latency, not by bandwidth).
// Padding up to a maximum that only the whole batch knows stays a launch of its own: letting the
// workgroup that finishes last do it (a ticket counter behind a device-scope fence) measured 39 us
// per call instead of 15, because such a fence writes back the L2 of the workgroup's XCD.  With
// `publish` there is nothing to pad afterwards (the rows are as far apart as the caller's guess,
// and padded that far here), and the maximum alone travels on atomics, with no fence: 8.8 us.
template <int K, bool LUT4_LDS, bool CHARS, bool HAS_MASK>
__global__ __launch_bounds__(kKmerThreads) void kmer_team_kernel(
    KmerArgs a, const uint8_t *__restrict__ bytes, const int64_t *__restrict__ offsets,
    int64_t n_rows, int64_t t_cap, int64_t fill_to, int32_t *__restrict__ ids,
    uint8_t *__restrict__ mask, int32_t *__restrict__ lengths, int32_t *__restrict__ status,
    int32_t *__restrict__ max_len, MaxRef mref, int publish)
{
    constexpr uint32_t POW4 = 1u << (2 * K);
    constexpr int NWV = kKmerThreads / 64;
    __shared__ uint32_t s_dig[256];
    __shared__ int32_t s_single[256];
    __shared__ __attribute__((aligned(16))) int32_t s_lut4[LUT4_LDS ? POW4 : 4];
    __shared__ int32_t s_spell[256];
    __shared__ __attribute__((aligned(16))) int32_t s_stage[NWV][kStageWords];
    __shared__ uint32_t s_tot[2][NWV];
    __shared__ int32_t s_stat[NWV];

    const int lane = threadIdx.x & 63;
    const int wv = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    // The kernel's life is a few trips to memory, so they are made to overlap: the bytes of the
    // workgroup's first row are requested first, then the tables (the id table with 16-byte loads,
    // all in flight together), and only then does anyone wait.
    uint32_t w_first[K];
#pragma unroll
    for (int i = 0; i < K; ++i) w_first[i] = 0;
    if ((int64_t)blockIdx.x < n_rows) {
        const int64_t row_start = offsets[blockIdx.x];
        const int len = (int)(offsets[blockIdx.x + 1] - row_start);
        const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<uint8_t *>(bytes + row_start), (short)0, len, 0x00020000);
        const int off = (wv * kWaveUnits + lane * kUnitsPerLane) * K;
        int i = 0;
#pragma unroll
        for (; i + 4 <= K; i += 4) {
            const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(rs, off + 4 * i, 0, 0);
            w_first[i] = v.x; w_first[i + 1] = v.y; w_first[i + 2] = v.z; w_first[i + 3] = v.w;
        }
        if (i + 2 <= K) {
            const u32x2 v = __builtin_amdgcn_raw_buffer_load_b64(rs, off + 4 * i, 0, 0);
            w_first[i] = v.x; w_first[i + 1] = v.y;
            i += 2;
        }
        if (i < K) w_first[i] = __builtin_amdgcn_raw_buffer_load_b32(rs, off + 4 * i, 0, 0);
    }
    if (LUT4_LDS) {
        constexpr int kVec = POW4 / 4;                               // 16-byte pieces of the id table
        constexpr int kPer = (kVec + kKmerThreads - 1) / kKmerThreads;
        const uint4 *src4 = reinterpret_cast<const uint4 *>(a.lut4);
        uint4 v[kPer];
#pragma unroll
        for (int q = 0; q < kPer; ++q) {
            const int at = (int)threadIdx.x + q * kKmerThreads;
            v[q] = at < kVec ? src4[at] : uint4{0, 0, 0, 0};
        }
        uint4 *dst4 = reinterpret_cast<uint4 *>(s_lut4);
#pragma unroll
        for (int q = 0; q < kPer; ++q) {
            const int at = (int)threadIdx.x + q * kKmerThreads;
            if (at < kVec) dst4[at] = v[q];
        }
    }
    for (int i = threadIdx.x; i < 256; i += kKmerThreads) {
        const int d = a.digit[i];
        s_dig[i] = d < 0 ? kDigBad : (d >= 4 ? kDigN : (uint32_t)d);
        s_single[i] = a.single[i];
        s_spell[i] = a.single[(int)"ACGTN"[d < 0 || d > 4 ? 4 : d]];
    }
    __syncthreads();

    int32_t *const buf = s_stage[wv];
    const int cap = t_cap > INT_MAX - 16 ? INT_MAX - 16 : (int)t_cap;
    const int fill = fill_to > cap ? cap : (int)fill_to;
    int64_t wg_max = 0;
    const unsigned long long slot_gen = mref.slot ? mref.slot[1] : 0ull;
    unsigned long long sent = 0, sent_val = 0;       // publish: the row's length + 1 and what its tree word held before

    for (int64_t row = blockIdx.x; row < n_rows; row += gridDim.x) {
        const int64_t row_start = offsets[row];
        const int len = (int)(offsets[row + 1] - row_start);
        const int full = len / K;
        const int n_units = full + (len - full * K);
        const uint8_t *src = bytes + row_start;
        int32_t *out = ids + row * t_cap;
        const int mis = (int)((reinterpret_cast<uintptr_t>(out) >> 2) & 3);
        int32_t *outA = out - mis;
        uint8_t *moutA = HAS_MASK ? mask + row * t_cap - mis : nullptr;
        const int hi_cap = mis + cap;
        int running = 0;
        int32_t my_status = 0;
        const __amdgpu_buffer_rsrc_t rsrc =
            __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t *>(src), (short)0, len, 0x00020000);
        if (publish && n_units == 0 && wv == 0 && lane == 0) {
            sent_val = 1;
            sent = atomicAdd(mref.tree + (blockIdx.x >> 2), 1ull << (16 * (blockIdx.x & 3)));
        }

        int par = 0;
        for (int r0 = 0; r0 < n_units; r0 += NWV * kWaveUnits, par ^= 1) {     // the same rounds for every wave
            const int u0 = r0 + wv * kWaveUnits;
            const int ub = u0 + lane * kUnitsPerLane;
            const bool lane_full = ub + kUnitsPerLane <= full;     // 4 whole windows
            const bool empty = ub >= n_units;
            uint32_t w[K];
            if (row == (int64_t)blockIdx.x && r0 == 0) {
#pragma unroll
                for (int i = 0; i < K; ++i) w[i] = w_first[i];
            } else {
                const int off = ub * K;                            // reads past the row's end return 0
                int i = 0;
#pragma unroll
                for (; i + 4 <= K; i += 4) {
                    const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(rsrc, off + 4 * i, 0, 0);
                    w[i] = v.x; w[i + 1] = v.y; w[i + 2] = v.z; w[i + 3] = v.w;
                }
                if (i + 2 <= K) {
                    const u32x2 v = __builtin_amdgcn_raw_buffer_load_b64(rsrc, off + 4 * i, 0, 0);
                    w[i] = v.x; w[i + 1] = v.y;
                    i += 2;
                }
                if (i < K) w[i] = __builtin_amdgcn_raw_buffer_load_b32(rsrc, off + 4 * i, 0, 0);
            }
            auto digit_of = [&](int bi) -> uint32_t { return s_dig[(w[bi >> 2] >> (8 * (bi & 3))) & 255u]; };
            uint32_t code[kUnitsPerLane];
            int32_t t[kUnitsPerLane];
#pragma unroll
            for (int j = 0; j < kUnitsPerLane; ++j) {
                uint32_t c = 0;
#pragma unroll
                for (int i = 0; i < K; ++i) c = (c << 2) + digit_of(j * K + i);
                code[j] = c;
                const uint32_t idx = c & (POW4 - 1);
                t[j] = LUT4_LDS ? s_lut4[idx] : a.lut4[idx];
            }
            const uint32_t any_flag = code[0] | code[1] | code[2] | code[3];
            const bool fast = lane_full && any_flag < POW4 && (t[0] | t[1] | t[2] | t[3]) >= 0;

            // tokens per unit and per lane (as in kmer_rows_kernel)
            int32_t cnt[kUnitsPerLane], ex[kUnitsPerLane], ey[kUnitsPerLane];
            uint32_t lane_cnt = 0;
            if (fast) {
                lane_cnt = kUnitsPerLane;
            } else if (lane_full) {
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
                    if (code[j] & kCodeBadBits) my_status |= DNATOK_ROW_INVALID_BYTE;
                    lane_cnt += (uint32_t)cnt[j];
                }
            } else if (!empty) {
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

            // where the wave's run starts: the steps of the waves before it in this round
            if (lane == 0) s_tot[par][wv] = step_total;
            __syncthreads();
            uint32_t before = 0, round_total = 0;
#pragma unroll
            for (int q = 0; q < NWV; ++q) {
                const uint32_t v = s_tot[par][q];
                before += q < wv ? v : 0u;
                round_total += v;
            }
            const int A = mis + running + (int)before;             // cell the step's first token goes to
            const int A_end = A + (int)step_total;
            const int lo = A, hi = A_end < hi_cap ? A_end : hi_cap;
            if (publish && wv == 0 && lane == 0 && r0 + NWV * kWaveUnits >= n_units) {
                // the row's length is known here, before its last tokens are written: the
                // maximum travels while they are (see the end of the kernel)
                const int total = running + (int)round_total;
                const int kept = total < cap ? total : cap;
                sent_val = (unsigned long long)kept + 1;
                sent = atomicAdd(mref.tree + (blockIdx.x >> 2), sent_val << (16 * (blockIdx.x & 3)));
            }
            const uint32_t carry = (uint32_t)A & 3u;
            const uint32_t n_avail = carry + step_total;
            const uint32_t s0 = carry + (inc - lane_cnt);
            const int e0 = A & ~3;

            auto produce = [&](auto put) {
                uint32_t s = s0;
                if (fast) {
#pragma unroll
                    for (int j = 0; j < kUnitsPerLane; ++j) put(s + j, t[j]);
                } else if (lane_full) {
#pragma unroll
                    for (int j = 0; j < kUnitsPerLane; ++j) {
                        if (code[j] < POW4 && t[j] >= 0) {
                            put(s, t[j]);
                            ++s;
                        } else if (CHARS) {
#pragma unroll
                            for (int i = 0; i < K; ++i) {
                                const int bi = j * K + i;
                                put(s + i, s_spell[(w[bi >> 2] >> (8 * (bi & 3))) & 255u]);
                            }
                            s += K;
                        } else if (ex[j] >= 0) {
                            put(s, ex[j]);
                            ++s;
                        } else if (ex[j] == INT_MIN) {
                            put(s, a.missing_id);
                            ++s;
                        } else {
                            for (int e = 0; e < -ex[j]; ++e) put(s + e, a.flat[ey[j] + e]);
                            s += -ex[j];
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
                                put(s, id);
                                ++s;
                            } else {
                                const int2 e = a.entry[c5];
                                if (e.x >= 0 || e.x == INT_MIN) {
                                    put(s, e.x >= 0 ? e.x : a.missing_id);
                                    ++s;
                                } else {
                                    for (int q = 0; q < -e.x; ++q) put(s + q, a.flat[e.y + q]);
                                    s += -e.x;
                                }
                            }
                        } else if (u < n_units) {
                            put(s, s_single[src[full * K + (u - full)]]);
                            ++s;
                        }
                    }
                }
            };
            // the staged run, written out in passes of kStageCap tokens (one pass unless a step
            // expands to more than that)
            for (uint32_t pass = 0; pass < n_avail; pass += kStageCap) {
                produce([&](uint32_t s, int32_t tok) {
                    const uint32_t rel = s - pass;
                    if (rel < (uint32_t)kStageCap) buf[rel] = tok;
                });
                wave_sync();
                const uint32_t count = pass + kStageCap >= n_avail ? n_avail - pass : (uint32_t)kStageCap;
                const uint32_t n_groups = (count + 3) >> 2;
                for (uint32_t g = lane; g < n_groups; g += 64) {
                    const int4v x = *reinterpret_cast<const int4v *>(buf + 4 * g);
                    const int32_t v[4] = {x.x, x.y, x.z, x.w};
                    store_group(outA, moutA, e0 + (int)pass + 4 * (int)g, lo, hi, v, 1u);
                }
                wave_sync();
            }
            running += (int)round_total;
        }

        // the row's end: length, status, padding (by the first wave)
        const bool any_bad = __ballot(my_status & DNATOK_ROW_INVALID_BYTE) != 0;
        const bool any_missing = __ballot(my_status & DNATOK_ROW_MISSING_KMER) != 0;
        if (lane == 0) s_stat[wv] = (any_bad ? DNATOK_ROW_INVALID_BYTE : 0) | (any_missing ? DNATOK_ROW_MISSING_KMER : 0);
        __syncthreads();
        const int stored = running < cap ? running : cap;
        if (wv == 0) {
            int32_t st = 0;
#pragma unroll
            for (int q = 0; q < NWV; ++q) st |= s_stat[q];
            if (running > t_cap) st |= DNATOK_ROW_TRUNCATED;
            if (lane == 0) {
                lengths[row] = (int32_t)running;
                if (status) status[row] = st;
            }
            if (fill > stored) pad_cells(outA, moutA, mis, stored, fill, a.pad_id, lane);
        }
        if (stored > wg_max) wg_max = stored;
        __syncthreads();                      // s_stat and s_tot are written again by the next row
    }
    if (wv == 0) {
        if (mref.slot && publish) {
            // the workgroup (it has one row: the grid is the batch) added its length + 1 to its tree
            // word as soon as the length was known, before the row's last tokens were written
            if (lane == 0) climb_max_tree(mref.tree, blockIdx.x, gridDim.x, sent_val, sent, max_len);
        } else if (mref.slot) {
            const unsigned long long v = (slot_gen << 32) | (unsigned long long)wg_max;
            if (lane == 0 && (wg_max > 0 || blockIdx.x == 0) && __builtin_nontemporal_load(mref.slot) < v)
                atomicMax(mref.slot, v);
        } else if (max_len && lane == 0 && wg_max > 0 && (int64_t)__builtin_nontemporal_load(max_len) < wg_max) {
            atomicMax(max_len, (int32_t)wg_max);
        }
    }
}

// Pads every row from its stored length up to the batch maximum found on the device.  A wave
// reads the lengths of kPadRows rows at once, then pads the rows that fall short one after
// the other, so that the stores of all of them are in flight together.
#ifndef DNATOK_PAD_ROWS
#define DNATOK_PAD_ROWS 8
#endif
constexpr int kPadRows = DNATOK_PAD_ROWS;

__global__ __launch_bounds__(256) void pad_to_max_kernel(
    int32_t *__restrict__ ids, uint8_t *__restrict__ mask, const int32_t *__restrict__ lengths,
    int64_t n_rows, int64_t t_cap, int32_t *__restrict__ max_len, int32_t pad_id, int32_t already, MaxRef mref)
{
    int fill;
    if (mref.slot) {
        // the maximum is in the call's slot; the slot's next user gets the next generation
        fill = (int)(uint32_t)mref.slot[0];
        if (blockIdx.x == 0 && threadIdx.x == 0) {
            *max_len = fill;
            mref.slot[1] = mref.slot[1] + 1;
        }
    } else {
        fill = *max_len;
    }
    if (fill <= already) return;          // every row is padded this far already
    const int lane = threadIdx.x & 63;
    const int64_t wave = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    const int64_t n_waves = (int64_t)gridDim.x * (blockDim.x >> 6);
    for (int64_t base = wave * kPadRows; base < n_rows; base += n_waves * kPadRows) {
        int len = fill;
        if (lane < kPadRows && base + lane < n_rows) {
            len = lengths[base + lane];
            if (len < already) len = already;
        }
        uint64_t todo = __ballot(len < fill);
        while (todo) {
            const int l = __builtin_ctzll(todo);
            todo &= todo - 1;
            const int from = __builtin_amdgcn_readlane(len, l);
            int32_t *out = ids + (base + l) * t_cap;
            const int mis = (int)((reinterpret_cast<uintptr_t>(out) >> 2) & 3);
            pad_cells(out - mis, mask ? mask + (base + l) * t_cap - mis : nullptr, mis, from, fill, pad_id, lane);
        }
    }
}

static int launch_pad(int32_t *ids, uint8_t *mask, const int32_t *lengths, int64_t n_rows, int64_t t_cap,
                      int32_t *max_len, int32_t pad_id, int32_t already, MaxRef mref, hipStream_t s)
{
    int64_t blocks = (n_rows + 4 * kPadRows - 1) / (4 * kPadRows);
    if (blocks > 256 * 16) blocks = 256 * 16;
    if (blocks < 1) blocks = 1;
    pad_to_max_kernel<<<(int)blocks, 256, 0, s>>>(ids, mask, lengths, n_rows, t_cap, max_len, pad_id, already, mref);
    DNATOK_HIP_TRY(hipGetLastError());
    return DNATOK_OK;
}

int launch_pad_to_max(int32_t *ids, uint8_t *mask, const int32_t *lengths, int64_t n_rows,
                      int64_t t_cap, int32_t *max_len, int32_t pad_id, int32_t already, hipStream_t s)
{
    return launch_pad(ids, mask, lengths, n_rows, t_cap, max_len, pad_id, already, MaxRef{nullptr, nullptr}, s);
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
    // The same ids in the order of the code that kmer_rows_kernel<..., ARITH> computes from the bytes
    // themselves: character i of the window in bits 2i, 2i + 1, as bits 1 and 2 of its ASCII code
    // (A 0, C 1, T 2, G 3).  That kernel serves the plain digit table: A C G T N -> 0 1 2 3 4, in
    // upper case alone or in both cases, every other byte outside the alphabet.
    std::vector<int32_t> lut4r(pow4);
    for (int64_t c4 = 0; c4 < pow4; ++c4) {
        int64_t r = 0;
        for (int i = 0; i < k; ++i) {
            const int64_t d = (c4 >> (2 * (k - 1 - i))) & 3;       // digit of character i
            r |= (d ^ (d >> 1)) << (2 * i);
        }
        lut4r[r] = lut4[c4];
    }
    bool plain_upper = true, plain_lower = true, no_lower = true;
    for (int b = 0; b < 256; ++b) {
        const char *u = strchr("ACGTN", b), *l = strchr("acgtn", b);
        const int want_u = (b && u) ? (int)(u - "ACGTN") : -1, want_l = (b && l) ? (int)(l - "acgtn") : -1;
        if (want_l >= 0) {
            plain_lower = plain_lower && digit_h[b] == want_l;
            no_lower = no_lower && digit_h[b] < 0;
        } else {
            plain_upper = plain_upper && (want_u < 0 ? digit_h[b] < 0 : digit_h[b] == want_u);
        }
    }
    const bool arith = plain_upper && (plain_lower || no_lower);
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
    const size_t o_lut4r = up(o_lut4 + pow4 * 4);
    const size_t o_entry = up(o_lut4r + pow4 * 4);
    const size_t o_flat = up(o_entry + pow5 * sizeof(int2));
    const size_t o_slots = up(o_flat + (has_exp ? n_flat * 4 : 0));
    const size_t o_trees = up(o_slots + (size_t)kMaxSlots * kMaxSlotStride * 8);
    const size_t bytes = up(o_trees + (size_t)kMaxSlots * kTreeWords * 8) + 256;
    std::vector<uint8_t> host(bytes, 0);
    memcpy(&host[o_digit], digit_h, 256);
    memcpy(&host[o_single], single_h, 256 * 4);
    memcpy(&host[o_lut4], lut4.data(), pow4 * 4);
    memcpy(&host[o_lut4r], lut4r.data(), pow4 * 4);
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
    t->lut4r = (int32_t *)(b + o_lut4r);
    t->arith = arith ? 1 : 0;
    t->fold = arith && plain_lower ? 0xDFDFDFDFu : 0xFFFFFFFFu;
    t->entry = (int2 *)(b + o_entry);
    t->flat = (int32_t *)(b + o_flat);
    t->max_slots = (unsigned long long *)(b + o_slots);
    t->max_trees = (unsigned long long *)(b + o_trees);
    *out = t;
    return DNATOK_OK;
}

extern "C" int dnatok_kmer_table_set_team_rows(dnatok_kmer_t *t, int32_t max_rows)
{
    DNATOK_REQUIRE(t, DNATOK_E_INVALID, "dnatok_kmer_table_set_team_rows: null table");
    DNATOK_REQUIRE(max_rows >= -1, DNATOK_E_INVALID, "dnatok_kmer_table_set_team_rows: -1 (automatic), 0 (never) or a row count");
    t->team_rows.store(max_rows, std::memory_order_relaxed);
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
    DNATOK_REQUIRE(n_rows >= 0 && t_cap >= 0 && fill_to <= t_cap, DNATOK_E_INVALID,
                   "dnatok_kmer_encode_padded: need fill_to <= t_cap");
    DNATOK_REQUIRE(fill_to > 0 || max_len, DNATOK_E_INVALID,
                   "dnatok_kmer_encode_padded: fill_to <= 0 needs max_len");
    // fill_to < 0: pad to the longest row; -fill_to is the caller's guess of that width.  Rows are
    // padded to the guess while they are written (next to the cells just stored, which is far
    // cheaper than coming back to every row), the pass after the kernel pads what is missing.
    const bool to_longest = fill_to <= 0;
    int64_t guess = to_longest ? -fill_to : 0;
    if (guess > t_cap) guess = t_cap;
    if (guess > INT_MAX - 16) guess = INT_MAX - 16;
    if (to_longest) fill_to = guess;
    if (n_rows == 0) return DNATOK_OK;
    hipStream_t s = (hipStream_t)stream;
    KmerArgs a{t->digit, t->single, t->lut4, t->lut4r, t->fold, t->entry, t->flat, t->pad_id, t->missing_id};
    MaxRef mref{nullptr, nullptr};
    if (to_longest) {
        std::lock_guard<std::mutex> hold(t->slot_lock);
        auto it = t->slot_of_stream.find(stream);
        if (it == t->slot_of_stream.end() && (int)t->slot_of_stream.size() < kMaxSlots)
            it = t->slot_of_stream.emplace(stream, (int)t->slot_of_stream.size()).first;
        if (it != t->slot_of_stream.end()) {
            mref.slot = t->max_slots + (size_t)it->second * kMaxSlotStride;
            mref.tree = t->max_trees + (size_t)it->second * kTreeWords;
        }
    }
    if (!mref.slot && max_len) {
        kmer_init_kernel<<<1, 1, 0, s>>>(max_len);
        DNATOK_HIP_TRY(hipGetLastError());
    }
    // persistent waves: the tables are staged into LDS once per workgroup
    const int64_t want = (n_rows + kRowsThreads / 64 - 1) / (kRowsThreads / 64);
    // few rows (a workgroup for every row at once): the four waves of a workgroup share a row.
    // When the row stride is already cut to the guess (at most kTightStride cells beyond it), the
    // rows are padded to the whole stride while they are written, which covers every possible
    // maximum: the kernel (either of the two) then reports the maximum itself and the padding
    // launch is left out (4 % of the 6-mer workload's step, 40 % of a single batch's).
    constexpr int64_t kTightStride = 256;
    const bool tight = to_longest && mref.slot && guess > 0 && t_cap - guess <= kTightStride && t_cap < 0xFFFF;
    bool padded_in_kernel = false;
    // short rows (a row stride of at most kGroupsMaxStride cells says so), the plain digit table,
    // every window without an id spelled by its characters: sixteen lanes per row
    const bool by_groups = t->arith && t->chars_mode && t_cap > 0 && t_cap <= kGroupsMaxStride && (t_cap & 3) == 0;
    if (by_groups) {
        padded_in_kernel = tight;
#define GROUPS2(KK, L, M)                                                                         \
    do {                                                                                          \
        static const int resident = resident_workgroups(kmer_groups_kernel<KK, L, M>, kGroupThreads, 0, 8); \
        int64_t grid = (n_rows + kGroupThreads / 16 - 1) / (kGroupThreads / 16);                  \
        if (grid > resident) grid = resident;                                                     \
        if (grid > kTreeRows) grid = kTreeRows;                                                   \
        kmer_groups_kernel<KK, L, M><<<(int)grid, kGroupThreads, 0, s>>>(                         \
            a, bytes, offsets, n_rows, t_cap, tight ? t_cap : fill_to, ids, mask, lengths, status, max_len, mref, \
            tight ? 1 : 0, RowPlace{nullptr, 0, 0});                                              \
    } while (0)
#define GROUPS(KK, L)                                                                             \
    do {                                                                                          \
        if (mask) GROUPS2(KK, L, true); else GROUPS2(KK, L, false);                               \
    } while (0)
        switch (t->k) {
            case 2: GROUPS(2, true); break;
            case 3: GROUPS(3, true); break;
            case 4: GROUPS(4, true); break;
            case 5: GROUPS(5, true); break;
            case 6: GROUPS(6, true); break;
            case 7: GROUPS(7, false); break;
            default: GROUPS(8, false); break;
        }
#undef GROUPS
#undef GROUPS2
    }
#define LAUNCH3(KK, L, C, M) \
    do {                                                                                          \
        if (t->arith) LAUNCH4(KK, L, C, M, true); else LAUNCH4(KK, L, C, M, false);               \
    } while (0)
#define LAUNCH4(KK, L, C, M, AR)                                                                  \
    do {                                                                                          \
        static const int resident = resident_workgroups(kmer_rows_kernel<KK, L, C, M, AR>, kRowsThreads, 0, 2); \
        static const int team_resident = resident_workgroups(kmer_team_kernel<KK, L, C, M>, kKmerThreads, 0, 4); \
        const int team_rows = t->team_rows.load(std::memory_order_relaxed);                         \
        if (n_rows <= (team_rows < 0 ? team_resident : team_rows)) {                              \
            padded_in_kernel = tight && n_rows <= kTreeRows;                                      \
            kmer_team_kernel<KK, L, C, M><<<(int)n_rows, kKmerThreads, 0, s>>>(                   \
                a, bytes, offsets, n_rows, t_cap, padded_in_kernel ? t_cap : fill_to, ids, mask,  \
                lengths, status, max_len, mref, padded_in_kernel ? 1 : 0);                        \
            break;                                                                                \
        }                                                                                         \
        const int64_t grid = want < resident ? want : resident;                                   \
        padded_in_kernel = tight && grid <= kTreeRows;                                            \
        kmer_rows_kernel<KK, L, C, M, AR><<<(int)grid, kRowsThreads, 0, s>>>(                     \
            a, bytes, offsets, n_rows, t_cap, padded_in_kernel ? t_cap : fill_to, ids, mask,      \
            lengths, status, max_len, mref, padded_in_kernel ? 1 : 0, RowPlace{nullptr, 0, 0});   \
    } while (0)
#define LAUNCH2(KK, L, C)                                                                         \
    do {                                                                                          \
        if (mask) LAUNCH3(KK, L, C, true); else LAUNCH3(KK, L, C, false);                         \
    } while (0)
#define LAUNCH(KK, L)                                                                             \
    do {                                                                                          \
        if (t->chars_mode) LAUNCH2(KK, L, true); else LAUNCH2(KK, L, false);                      \
    } while (0)
    if (!by_groups) switch (t->k) {
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
#undef LAUNCH3
#undef LAUNCH4
    DNATOK_HIP_TRY(hipGetLastError());
    if (to_longest && !padded_in_kernel)
        return launch_pad(ids, mask, lengths, n_rows, t_cap, max_len, t->pad_id, (int32_t)guess, mref, s);
    return DNATOK_OK;
}

// ---- rows placed by the caller's layout: row classes, packed output ------------------------------

namespace dnatok {
int launch_scan_lengths(const int32_t *lengths, int64_t n_rows, int64_t *out_offsets, void *scratch,
                        size_t scratch_bytes, hipStream_t s);   // pack.hip
}

// One launch of kmer_rows_kernel<..., PLACED> (which = 0) or kmer_groups_kernel (which = 1) with a
// RowPlace.  The longest row, where asked for, goes to mref.slot / max_len by atomicMax (no tree:
// two launches may share one call).
static int launch_placed(const dnatok_kmer_t *t, int which, const uint8_t *bytes, const int64_t *offsets, int64_t n_rows,
                         int64_t t_cap, int64_t fill_to, int32_t *ids, uint8_t *mask, int32_t *lengths,
                         int32_t *status, int32_t *max_len, MaxRef mref, RowPlace place, hipStream_t s)
{
    KmerArgs a{t->digit, t->single, t->lut4, t->lut4r, t->fold, t->entry, t->flat, t->pad_id, t->missing_id};
    if (which == 1) {
#define PG2(KK, L, M)                                                                              \
    do {                                                                                          \
        static const int resident = resident_workgroups(kmer_groups_kernel<KK, L, M>, kGroupThreads, 0, 8); \
        int64_t grid = (n_rows + kGroupThreads / 16 - 1) / (kGroupThreads / 16);                  \
        if (grid > resident) grid = resident;                                                     \
        kmer_groups_kernel<KK, L, M><<<(int)grid, kGroupThreads, 0, s>>>(                         \
            a, bytes, offsets, n_rows, t_cap, fill_to, ids, mask, lengths, status, max_len, mref, 0, place); \
    } while (0)
#define PG(KK, L)                                                                                 \
    do {                                                                                          \
        if (mask) PG2(KK, L, true); else PG2(KK, L, false);                                       \
    } while (0)
        switch (t->k) {
            case 2: PG(2, true); break;
            case 3: PG(3, true); break;
            case 4: PG(4, true); break;
            case 5: PG(5, true); break;
            case 6: PG(6, true); break;
            case 7: PG(7, false); break;
            default: PG(8, false); break;
        }
#undef PG
#undef PG2
    } else {
        const int64_t want = (n_rows + kRowsThreads / 64 - 1) / (kRowsThreads / 64);
#define PR4(KK, L, C, M, AR)                                                                      \
    do {                                                                                          \
        static const int resident = resident_workgroups(kmer_rows_kernel<KK, L, C, M, AR, true>, kRowsThreads, 0, 2); \
        const int64_t grid = want < resident ? want : resident;                                   \
        kmer_rows_kernel<KK, L, C, M, AR, true><<<(int)grid, kRowsThreads, 0, s>>>(               \
            a, bytes, offsets, n_rows, t_cap, fill_to, ids, mask, lengths, status, max_len, mref, 0, place); \
    } while (0)
#define PR3(KK, L, C, M)                                                                          \
    do {                                                                                          \
        if (t->arith) PR4(KK, L, C, M, true); else PR4(KK, L, C, M, false);                       \
    } while (0)
#define PR2(KK, L, C)                                                                             \
    do {                                                                                          \
        if (mask) PR3(KK, L, C, true); else PR3(KK, L, C, false);                                 \
    } while (0)
#define PR(KK, L)                                                                                 \
    do {                                                                                          \
        if (t->chars_mode) PR2(KK, L, true); else PR2(KK, L, false);                              \
    } while (0)
        switch (t->k) {
            case 2: PR(2, true); break;
            case 3: PR(3, true); break;
            case 4: PR(4, true); break;
            case 5: PR(5, true); break;
            case 6: PR(6, true); break;
            case 7: PR(7, false); break;
            default: PR(8, false); break;
        }
#undef PR
#undef PR2
#undef PR3
#undef PR4
    }
    DNATOK_HIP_TRY(hipGetLastError());
    return DNATOK_OK;
}

// A batch of mostly short rows (the mean at most kGroupsMaxUnits units) whose table the 16-lane
// kernel serves: that kernel takes the rows of at most kGroupsMaxUnits units, a wave per row the
// others.  (The row's class is read from its length on the device; what the host knows is the mean.)
static bool split_by_row_class(const dnatok_kmer_t *t, int64_t n_rows, int64_t total)
{
    return t->arith && t->chars_mode && n_rows > 0 && total / n_rows <= (int64_t)kGroupsMaxUnits * t->k;
}

extern "C" int dnatok_kmer_encode_padded_sized(const dnatok_kmer_t *t, const uint8_t *bytes, const int64_t *offsets,
                                               int64_t n_rows, int64_t total, int64_t t_cap, int64_t fill_to,
                                               int32_t *ids, uint8_t *mask, int32_t *lengths, int32_t *status,
                                               int32_t *max_len, void *stream)
{
    DNATOK_REQUIRE(t && offsets && ids && lengths, DNATOK_E_INVALID, "dnatok_kmer_encode_padded_sized: null argument");
    DNATOK_REQUIRE(n_rows >= 0 && total >= 0 && t_cap >= 0 && fill_to <= t_cap, DNATOK_E_INVALID,
                   "dnatok_kmer_encode_padded_sized: need fill_to <= t_cap and sizes >= 0");
    DNATOK_REQUIRE(fill_to > 0 || max_len, DNATOK_E_INVALID, "dnatok_kmer_encode_padded_sized: fill_to <= 0 needs max_len");
    // A stride within the 16-lane kernel's reach says that every row is short; a batch of few rows,
    // or of rows that are long on average, is as well off with one kernel for all of them.
    const int team_rows = t->team_rows.load(std::memory_order_relaxed);
    if (n_rows < 1024 || t_cap <= kGroupsMaxStride || (t_cap & 3) != 0 || team_rows != -1 ||
        !split_by_row_class(t, n_rows, total))
        return dnatok_kmer_encode_padded(t, bytes, offsets, n_rows, t_cap, fill_to, ids, mask, lengths, status, max_len,
                                         stream);
    const bool to_longest = fill_to <= 0;
    int64_t guess = to_longest ? -fill_to : 0;
    if (guess > t_cap) guess = t_cap;
    if (to_longest) fill_to = guess;
    hipStream_t s = (hipStream_t)stream;
    MaxRef mref{nullptr, nullptr};
    if (to_longest) {
        std::lock_guard<std::mutex> hold(t->slot_lock);
        auto it = t->slot_of_stream.find(stream);
        if (it == t->slot_of_stream.end() && (int)t->slot_of_stream.size() < kMaxSlots)
            it = t->slot_of_stream.emplace(stream, (int)t->slot_of_stream.size()).first;
        if (it != t->slot_of_stream.end()) {
            mref.slot = t->max_slots + (size_t)it->second * kMaxSlotStride;
            mref.tree = t->max_trees + (size_t)it->second * kTreeWords;
        }
        if (!mref.slot) {
            kmer_init_kernel<<<1, 1, 0, s>>>(max_len);
            DNATOK_HIP_TRY(hipGetLastError());
        }
    }
    int rc = launch_placed(t, 1, bytes, offsets, n_rows, t_cap, fill_to, ids, mask, lengths, status, max_len, mref,
                           RowPlace{nullptr, 1, 0}, s);
    if (rc) return rc;
    rc = launch_placed(t, 0, bytes, offsets, n_rows, t_cap, fill_to, ids, mask, lengths, status, max_len, mref,
                       RowPlace{nullptr, 2, 0}, s);
    if (rc) return rc;
    if (to_longest) return launch_pad(ids, mask, lengths, n_rows, t_cap, max_len, t->pad_id, (int32_t)guess, mref, s);
    return DNATOK_OK;
}

extern "C" int dnatok_kmer_encode_packed(const dnatok_kmer_t *t, const uint8_t *bytes, const int64_t *offsets,
                                         int64_t n_rows, int64_t total, int32_t *ids_out, int64_t *out_offsets,
                                         uint8_t *mask_out, int32_t *lengths, int32_t *status, void *stream)
{
    DNATOK_REQUIRE(t && offsets && out_offsets && lengths, DNATOK_E_INVALID, "dnatok_kmer_encode_packed: null argument");
    DNATOK_REQUIRE(n_rows >= 0 && total >= 0, DNATOK_E_INVALID, "dnatok_kmer_encode_packed: negative size");
    DNATOK_REQUIRE(ids_out || total == 0, DNATOK_E_INVALID, "dnatok_kmer_encode_packed: null ids_out");
    hipStream_t s = (hipStream_t)stream;
    const bool split = split_by_row_class(t, n_rows, total);
    const MaxRef none{nullptr, nullptr};
    // first pass: every row's token count (nothing else is written), then where every row starts
    if (n_rows > 0) {
        int rc;
        if (split) {
            rc = launch_placed(t, 1, bytes, offsets, n_rows, 0, 0, nullptr, nullptr, lengths, nullptr, nullptr, none,
                               RowPlace{nullptr, 1, 1}, s);
            if (rc) return rc;
        }
        rc = launch_placed(t, 0, bytes, offsets, n_rows, 0, 0, nullptr, nullptr, lengths, nullptr, nullptr, none,
                           RowPlace{nullptr, split ? 2 : 0, 1}, s);
        if (rc) return rc;
    }
    // (ids_out is not written yet: its first bytes, when 8-byte aligned, are the scan's spare room)
    int rc = launch_scan_lengths(lengths, n_rows, out_offsets, ids_out, (size_t)total * 4, s);
    if (rc || n_rows == 0) return rc;
    // second pass: the tokens, each row behind the one before it
    if (split) {
        rc = launch_placed(t, 1, bytes, offsets, n_rows, 0, 0, ids_out, mask_out, lengths, status, nullptr, none,
                           RowPlace{out_offsets, 1, 0}, s);
        if (rc) return rc;
    }
    return launch_placed(t, 0, bytes, offsets, n_rows, 0, 0, ids_out, mask_out, lengths, status, nullptr, none,
                         RowPlace{out_offsets, split ? 2 : 0, 0}, s);
}
