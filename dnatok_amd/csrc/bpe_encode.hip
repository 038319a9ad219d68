// BPE merge engine: reproduces the Hugging Face word-merge order exactly.
//
// HF pops adjacent pairs from a heap keyed (rank, position), skips stale entries, merges, and
// pushes the two new neighbour pairs.  That is "always merge the pair with the smallest
// (rank, position) key".  The engine below gets the same result in rounds:
//
//   * every live position i keeps the rank R[i] of the pair it starts; a team of threads
//     (one wave, or one workgroup) finds rmin = min R and the gate G = min over current
//     pairs of gate(R[i]), where gate(r) is the lowest rank of any rule that uses the
//     symbol rule r creates.  No pair born in this round can have a rank below G, so all
//     current pairs with rank in [rmin, G) can be settled together;
//   * among those candidates a pair merges unless an overlapping candidate with a smaller
//     key merges.  Overlaps form chains of strictly decreasing key, along which the decision
//     alternates, so each candidate walks its left and right chain and merges iff both have
//     even length (for a run x x x x this is "every other one from the left", HF's tie rule);
//   * the candidates of a round go onto a queue and are dealt one per thread for these walks (the
//     threads find them among their own positions from ranks they keep in registers); the pairs
//     that merge go onto a second queue, which deals the apply work (one merge per thread) and the
//     re-rank work (two table lookups per merge) evenly to the team, whatever positions the merges
//     sit at.  Merges are applied in a doubly linked list over the original
//     positions (a merge keeps the left position); rank, links and symbol of a position sit in one
//     record, so a step along a chain is one read; the two neighbour pairs of each new symbol are
//     re-ranked through the hashed merge table, and only the threads whose positions changed
//     refresh their cached minima.
//
// A table in which some rule's product is used by a LOWER-ranked rule (possible when two
// rules produce the same string) makes G <= rmin; such a round merges only the single
// smallest-key pair, which is exactly HF's next step.
//
// State lives in LDS for rows up to the LDS capacity (15 bytes per position: an 8-byte record,
// product and gate of the position's pair, and the two queues), and in a global scratch area
// (L2-resident, 32-bit links) for longer rows that cannot be cut into chunks.
#include "common.hpp"

#include <stdlib.h>
#include <string.h>
#include <atomic>
#include <mutex>
#include <unordered_map>
#include <vector>

struct dnatok_bpe_table {
    int32_t n_merges, n_symbols;
    uint32_t slots, shift;       // hash table size (power of two) and 32 - log2(slots)
    uint32_t mul1, mul2;         // multipliers of the two hash functions
    int monotone;                // no rule's product is used by a lower-ranked rule
    void *blob;
    uint4 *tab;                  // [slots]  {key = a << 16 | b, rank, product | gate << 16, 0}
    uint16_t *byte_to_sym;       // [256]
    int32_t *out_remap;          // [n_symbols] or nullptr
    uint32_t *ltab;              // the compact form of the table that fits LDS (kLdsTabWords words), or nullptr
    uint32_t lmul1, lmul2;       // its two multipliers
    void *first;                 // dnatok::FirstPairs on the device, or nullptr (more bytes with rules than classes)
    // dnatok_bpe_encode_padded: the tree of atomics that carries a call's longest row
    // (dnatok::publish_max), one per stream that encodes with this table (calls on one stream are
    // ordered, calls on different streams may overlap); a stream beyond the kMaxTreeSlots-th gets
    // its maximum from a launch over the lengths instead
    unsigned long long *max_trees;
    mutable std::mutex slot_lock;
    mutable std::unordered_map<void *, int> slot_of_stream;
    // Test and measurement switches of this table (dnatok_bpe_table_set_chunk_geometry,
    // dnatok_bpe_table_set_placement); 0 / 0 / 0 are the shipped choices.  A call reads them once,
    // when it starts.
    std::atomic<int> chunk_core{0}, chunk_overlap{0}, placement{0};
};

constexpr int kMaxTreeSlots = 64;

namespace dnatok {

constexpr uint32_t kNone = 0xFFFFu;          // "no rule" rank / dead symbol
constexpr uint32_t kEmptyKey = 0xFFFFFFFFu;

struct BpeArgs {
    const uint4 *tab;
    const uint16_t *byte_to_sym;
    const int32_t *out_remap;
    uint32_t shift, mul1, mul2;
    int32_t n_merges;
    const uint32_t *ltab;
    uint32_t lmul1, lmul2;
    const void *first;           // FirstPairs (global memory) or nullptr
    // single-character ids of the same bytes, written in the same pass (dnatok_bpe_encode_with_chars):
    // char_ids[i] = char_lut[bytes[i]], char_mask[i] = 1 (null: no mask)
    const int32_t *char_lut;
    int32_t *char_ids;
    uint8_t *char_mask;
    // rows padded in the same pass (dnatok_bpe_encode_padded; pad_ids = null: not asked for): row b's
    // ids go to pad_ids[b * pad_stride ..], through pad_remap when given, pad_id behind them up to
    // the stride, 1 / 0 to pad_mask (null: no mask); the longest row's token count goes up max_tree
    // (null: the caller finds it from the lengths) into *longest
    void *pad_ids;               // [n_rows, pad_stride] of pad_elem-byte integers (1, 2, 4 or 8)
    int32_t pad_elem, pad_left;  // pad_left: a row's tokens end at its last cell instead of starting at its first
    uint8_t *pad_mask;
    const int32_t *pad_remap;
    int64_t pad_stride;
    int32_t pad_id;
    unsigned long long *max_tree;
    int32_t *longest;
    // the work list holds no rows: item i is row i (bpe_plan_in_order_kernel)
    int32_t in_order;
    // items a team takes from its work counter at a time, and the counters in use (a power of two,
    // at most kDealers and at most the number of teams: every counter needs a team)
    int32_t grab, dealers;
    // which part of the work list a launch works through: 0 all of it, 1 all but the class of the
    // shortest rows, 2 that class alone (a batch of mostly short rows with a few long ones is split
    // between a launch with 256-thread teams and one with teams of one wave)
    int32_t part;
    // host side only: where the merge table is kept (dnatok_bpe_table_set_placement)
    int32_t placement;
};

// The arguments of the running kernel where they lie in memory.  What a kernel needs once per row
// and late (where a padded row goes, what pads it) is read from there at that point, after the
// merges, instead of held in registers all through them: a register more during the merges is a
// team less per CU at the sizes that count.
typedef const __attribute__((address_space(4))) BpeArgs *BpeArgsInMemory;

// (the pointer's halves go through an empty asm statement, so that the reads behind it stay where
// they are written instead of being moved to the kernel's start)
__device__ __forceinline__ BpeArgsInMemory kernel_args_now()
{
    const uintptr_t at = (uintptr_t)__builtin_amdgcn_kernarg_segment_ptr();
    uint32_t lo = (uint32_t)at, hi = (uint32_t)(at >> 32);
    asm volatile("" : "+v"(lo), "+v"(hi));
    lo = __builtin_amdgcn_readfirstlane(lo);
    hi = __builtin_amdgcn_readfirstlane(hi);
    return (BpeArgsInMemory)(((uintptr_t)hi << 32) | lo);
}

typedef int32_t bpe_int4_a4 __attribute__((ext_vector_type(4), aligned(4)));
typedef uint32_t bpe_u32_a1 __attribute__((aligned(1)));

// What a position keeps about the pair it starts: the rule's rank (kNone = no rule), the
// symbol the rule produces, and the rule's gate (lowest rank of any rule using that product).
struct PairInfo {
    uint32_t rank, pg;           // pg: the rule's product | its gate << 16, as the tables and the state hold them
};
constexpr uint32_t kNoPg = kNone | (kNone << 16);

// The rules between two single-byte symbols, by the bytes themselves: what every position of a row
// needs first.  A DNA alphabet has a handful of bytes with such rules (A C G T N), so the bytes are
// put into at most kFirstClasses classes and the rule of a pair of classes is one 8-byte read from
// a table a workgroup keeps in LDS, where the general table costs two reads from L2 behind two
// hashes (11 % of a 1 KB row's time went into its first pairs).  A table with more such bytes than
// classes has no FirstPairs and every lookup goes to the general table.
// The table takes the place of the byte-to-symbol table in a workgroup's LDS (a class knows its
// symbol; the symbol of a byte without a class is read from memory): 144 bytes more, not 768.
// LDS is handed out in pieces of kLdsPiece bytes, 128 per CU, and the forms for 2 KB chunks and for
// four rows of 512 bytes sit 304 and 256 bytes under a piece boundary: beyond it a CU holds four
// workgroups instead of five (measured: a batch of 100 kbp rows 13 % slower).
constexpr int kFirstClasses = 8;
constexpr uint32_t kNoClass = 15;
struct FirstPairs {
    uint8_t cls4[128];                                  // the byte's class, 4 bits each (low nibble: even byte); kNoClass: no rule pairs it with another byte
    uint16_t sym[kFirstClasses];                        // the class's symbol
    uint2 rule[kFirstClasses * kFirstClasses];          // [left class * 8 + right class] {rank, product | gate << 16}; rank kNone: no rule
    __device__ __forceinline__ uint32_t cls(uint32_t byte) const { return (cls4[byte >> 1] >> ((byte & 1u) * 4u)) & 15u; }
};
constexpr int kLdsPiece = 1280, kLdsPieces = 128;
// what a workgroup keeps of the table's small parts: FirstPairs, or the byte-to-symbol table
constexpr size_t kLeadBytes = sizeof(FirstPairs) > 512 ? sizeof(FirstPairs) : 512;

// The merge table is a cuckoo hash: every rule sits in one of the two slots its key hashes to, so
// a lookup is two independent reads issued together and never a chain of dependent ones.  (With
// linear probing a wave's lookup was as slow as its unluckiest lane: two to three trips to L2 per
// lookup even at one rule per eight slots.)
struct PairTable {
    const uint4 *tab;
    uint32_t shift, mul1, mul2;
};

struct PairEntry {               // the three words of a slot that carry something
    uint32_t x, y, z;
};

struct PairProbe {
    PairEntry e1, e2;
};

__host__ __device__ __forceinline__ uint32_t pair_slot(uint32_t key, uint32_t mul, uint32_t shift)
{
    return (key * mul) >> shift;
}

// Both reads of the rule for (a, b); issued for several pairs back to back, so that their memory
// latencies overlap.  pair_finish picks the answer.
__device__ __forceinline__ PairProbe pair_probe(const PairTable &t, uint32_t a, uint32_t b)
{
    const uint32_t key = (a << 16) | b;
    PairProbe pr;
    pr.e1 = *reinterpret_cast<const PairEntry *>(t.tab + pair_slot(key, t.mul1, t.shift));
    pr.e2 = *reinterpret_cast<const PairEntry *>(t.tab + pair_slot(key, t.mul2, t.shift));
    return pr;
}

__device__ __forceinline__ PairInfo pair_finish(uint32_t a, uint32_t b, const PairProbe &pr)
{
    const uint32_t key = (a << 16) | b;
    const bool first = pr.e1.x == key;
    const uint32_t y = first ? pr.e1.y : pr.e2.y, z = first ? pr.e1.z : pr.e2.z;
    if (!first && pr.e2.x != key) return PairInfo{kNone, kNoPg};
    return PairInfo{y, z};
}

// The compact form of the merge table, for tables of at most 8192 symbols and 4095 rules: small
// enough (48 KB) for a workgroup to keep in LDS when a batch leaves that much room.  A pair's key has
// 26 bits (two 13-bit symbols); key * odd multiplier mod 2^26 is a bijection, whose upper 13 bits are
// the slot and whose lower 13 bits are kept in the slot, together with which of the two functions
// placed the rule there: slot number, remainder and function give the key back, so a matching
// remainder is a matching key.  Slot word: rank << 15 | remainder << 2 | function << 1 | 1 (0 = empty).
// Product and gate of a rule are looked up by its rank in a second array.
constexpr int kLdsTabSlots = 8192;
constexpr int kLdsTabRanks = 4096;
constexpr int kLdsTabWords = kLdsTabSlots + kLdsTabRanks;      // 48 KB

struct LdsPairTable {
    const uint32_t *tab;         // [kLdsTabSlots], in LDS
    const uint32_t *pg;          // [kLdsTabRanks] product | gate << 16, in LDS
    uint32_t mul1, mul2;
};

struct LdsPairProbe {
    uint32_t e1, e2, want1, want2;
};

__host__ __device__ __forceinline__ uint32_t lds_pair_hash(uint32_t key24, uint32_t mul)
{
    return (key24 * mul) & 0x3FFFFFFu;
}

__device__ __forceinline__ LdsPairProbe pair_probe(const LdsPairTable &t, uint32_t a, uint32_t b)
{
    const uint32_t key = ((a & 0x1FFFu) << 13) | (b & 0x1FFFu);
    const uint32_t h1 = lds_pair_hash(key, t.mul1), h2 = lds_pair_hash(key, t.mul2);
    LdsPairProbe pr;
    pr.e1 = t.tab[h1 >> 13];
    pr.e2 = t.tab[h2 >> 13];
    pr.want1 = ((h1 & 0x1FFFu) << 2) | 1u;
    pr.want2 = ((h2 & 0x1FFFu) << 2) | 3u;
    return pr;
}

__device__ __forceinline__ PairInfo pair_finish(const LdsPairTable &t, uint32_t, uint32_t, const LdsPairProbe &pr)
{
    const bool first = (pr.e1 & 0x7FFFu) == pr.want1;
    if (!first && (pr.e2 & 0x7FFFu) != pr.want2) return PairInfo{kNone, kNoPg};
    const uint32_t rank = (first ? pr.e1 : pr.e2) >> 15;
    return PairInfo{rank, t.pg[rank]};
}

__device__ __forceinline__ PairInfo pair_finish(const PairTable &, uint32_t a, uint32_t b, const PairProbe &pr)
{
    return pair_finish(a, b, pr);
}

template <int NT>
__device__ __forceinline__ void team_sync()
{
    if (NT == 64) {
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
    } else {
        __syncthreads();
    }
}

// Minimum of two values over the team; includes exactly one team_sync.
template <int NT>
__device__ __forceinline__ void team_min2(uint32_t a, uint32_t b, uint32_t *red, int wv,
                                          uint32_t &ra, uint32_t &rb)
{
    a = wave_min_u32(a);
    b = wave_min_u32(b);
    if (NT == 64) {
        team_sync<NT>();
        ra = a; rb = b;
        return;
    }
    constexpr int NW = NT / 64;
    if ((threadIdx.x & 63) == 0) { red[wv * 2] = a; red[wv * 2 + 1] = b; }
    __syncthreads();
    uint32_t x = kEmptyKey, y = kEmptyKey;
#pragma unroll
    for (int w = 0; w < NW; ++w) { x = umin(x, red[w * 2]); y = umin(y, red[w * 2 + 1]); }
    ra = x; rb = y;
}

// The same for two values below 2^16 (ranks, gates and positions of pieces that fit LDS; anything
// above counts as 0xFFFF): both ride in one register, and one packed 16-bit minimum per step
// reduces them together.  Half the vector instructions of the two separate reductions, in a
// kernel that is bound by their number.
typedef unsigned short bpe_u16x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ uint32_t pk_min_u16(uint32_t a, uint32_t b)
{
    return __builtin_bit_cast(uint32_t, __builtin_elementwise_min(__builtin_bit_cast(bpe_u16x2, a),
                                                                  __builtin_bit_cast(bpe_u16x2, b)));
}

template <int NT>
__device__ __forceinline__ void team_min2_u16(uint32_t a, uint32_t b, uint32_t *red, int wv,
                                              uint32_t &ra, uint32_t &rb)
{
    uint32_t v = umin(a, 0xFFFFu) | (umin(b, 0xFFFFu) << 16);
    v = pk_min_u16(v, dpp_u32<0xB1>(v));    // quad_perm [1,0,3,2]
    v = pk_min_u16(v, dpp_u32<0x4E>(v));    // quad_perm [2,3,0,1]
    v = pk_min_u16(v, dpp_u32<0x141>(v));   // row_half_mirror
    v = pk_min_u16(v, dpp_u32<0x140>(v));   // row_mirror
    const uint32_t r0 = __builtin_amdgcn_readlane(v, 0), r1 = __builtin_amdgcn_readlane(v, 16);
    const uint32_t r2 = __builtin_amdgcn_readlane(v, 32), r3 = __builtin_amdgcn_readlane(v, 48);
    v = pk_min_u16(pk_min_u16(r0, r1), pk_min_u16(r2, r3));
    if (NT == 64) {
        team_sync<NT>();
    } else {
        constexpr int NW = NT / 64;
        if ((threadIdx.x & 63) == 0) red[wv] = v;
        __syncthreads();
        v = red[0];
#pragma unroll
        for (int w = 1; w < NW; ++w) v = pk_min_u16(v, red[w]);
    }
    ra = v & 0xFFFFu; rb = v >> 16;
}

// Number of set bits of a ballot below the calling lane (two instructions; written as a popcount
// of the ballot under a mask of the lower lanes it is four, and the engine is bound by their number).
__device__ __forceinline__ uint32_t lanes_below(uint64_t ballot)
{
    return __builtin_amdgcn_mbcnt_hi((uint32_t)(ballot >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)ballot, 0u));
}

// Exclusive prefix sum over the team (one value per thread) and the team total.
template <int NT>
__device__ __forceinline__ uint32_t team_exclusive_sum(uint32_t v, uint32_t *red, int wv, uint32_t &total)
{
    const uint32_t inc = wave_inclusive_sum_u32(v);
    if (NT == 64) {
        total = __builtin_amdgcn_readlane(inc, 63);
        return inc - v;
    }
    constexpr int NW = NT / 64;
    if ((threadIdx.x & 63) == 63) red[wv] = inc;
    __syncthreads();
    uint32_t carry = 0, tot = 0;
#pragma unroll
    for (int w = 0; w < NW; ++w) { const uint32_t t = red[w]; if (w < wv) carry += t; tot += t; }
    __syncthreads();
    total = tot;
    return carry + inc - v;
}

// Where a team's time goes, phase by phase: a build option (-DDNATOK_BPE_PHASE_CYCLES: the library
// libdnatok_hip_phases.so, never the product library, whose PhaseClock is empty and costs nothing).
// Thread 0 of every team reads the shader clock at the end of each phase of bpe_row and adds the
// cycles since the last reading to the phase's cell; a barrier at the end of a phase counts for
// that phase.  The cells of a workgroup (kPhaseCells each, workgroups modulo kPhaseGroups) are read
// and cleared by dnatok_bpe_phase_cycles.  The instrumented kernels hold more registers than the
// shipped ones (fewer teams per CU): the shares of the phases are what the numbers are for.
enum BpePhase {
    kPhInitial = 0, kPhMinimum, kPhCollect, kPhDecide, kPhLate, kPhApply, kPhRerank, kPhRefresh, kPhOutput,
    kPhRounds = 12, kPhMerges = 13, kPhPositions = 14, kPhItems = 15, kPhaseCells = 16
};
#ifdef DNATOK_BPE_PHASE_CYCLES
constexpr int kPhaseGroups = 4096;
__device__ unsigned long long g_phase_cycles[kPhaseGroups * kPhaseCells];
struct PhaseClock {
    long long t, cell[kPhaseCells];
    __device__ __forceinline__ PhaseClock() : t(clock64())
    {
#pragma unroll
        for (int q = 0; q < kPhaseCells; ++q) cell[q] = 0;
    }
    __device__ __forceinline__ void lap(const int phase)
    {
        const long long now = clock64();
        cell[phase] += now - t;
        t = now;
    }
    __device__ __forceinline__ void count(const int what, const long long n) { cell[what] += n; }
    __device__ __forceinline__ void flush(const int tid)
    {
        if (tid != 0) return;
        unsigned long long *g = g_phase_cycles + (size_t)(blockIdx.x % kPhaseGroups) * kPhaseCells;
#pragma unroll
        for (int q = 0; q < kPhaseCells; ++q)
            if (cell[q]) atomicAdd(&g[q], (unsigned long long)cell[q]);
    }
};
#else
struct PhaseClock {
    __device__ __forceinline__ void lap(int) {}
    __device__ __forceinline__ void count(int, long long) {}
    __device__ __forceinline__ void flush(int) {}
};
#endif

// What the engine keeps per position, in one record so that a step along a chain of candidates
// is one read: rank of the pair the position starts (kNone = no rule / dead), right and left
// live neighbour, symbol.  8 bytes with 16-bit links (LDS kernels), 16 bytes with 32-bit links
// (whole-row kernel, state in global memory).
template <typename IT>
struct alignas(4 * sizeof(IT)) PosRec {
    IT r, nx, pv, s;
};

// One row.  tid = index in the team; P and PG (product and gate of the pair a position starts) hold
// n0 entries, Q (the merges of the current round)
// n0 / 2, C (its candidates) n0; D holds NT bytes; PER > 0 says that n0 <= PER * NT, and every thread
// then keeps the ranks of its own positions in registers as well; red holds 4 * (NT / 64) + 4 words.  Tokens go to out[0 .. *out_len).
// CHARS: while the piece's bytes pass through the registers on their way into LDS, the
// single-character id of every byte in [char_lo, char_hi) is written to char_ids (and 1 to char_mask,
// when given); both pointers are those of the piece's byte 0.
// pad_stride > 0: out is a row of pad_stride cells; tokens beyond it are dropped (the count handed
// back is that of all tokens), the cells behind the tokens get pad_id, pad_mask (when given) 1 for
// a token and 0 for padding, and ids pass through remap2 (when given) after out_remap.
// Returns the row's token count (0 for a chunk).
template <int NT, typename IT, int PER, bool CHARS = false, bool PAD = false, typename PT>
__device__ __forceinline__ int32_t bpe_row(
    const PT pt, const uint16_t *byte_to_sym,
    const int32_t *out_remap, const uint8_t *__restrict__ src, const int n0, PosRec<IT> *P,
    uint32_t *PG, IT *Q, IT *C, uint8_t *D, uint32_t *red, const int tid,
    int32_t *__restrict__ out, int32_t *__restrict__ out_len, uint16_t *__restrict__ raw_out = nullptr,
    const int mid_lo = 0, const int mid_hi = 0, int32_t *__restrict__ mid_out = nullptr,
    const int32_t *__restrict__ char_lut = nullptr, int32_t *__restrict__ char_ids = nullptr,
    uint8_t *__restrict__ char_mask = nullptr, const int char_lo = 0, const int char_hi = 0,
    const FirstPairs *first = nullptr, const int32_t pad_row = 0,
    const uint16_t *__restrict__ byte_to_sym_far = nullptr)
{
    static_assert(!CHARS || PER > 0, "the single-character ids are written from the staged bytes");
    constexpr IT NIL = (IT)~(IT)0;
    constexpr IT DEAD = (IT)kNone;
    // pairs of table reads in flight per thread.  (Two cost eight registers, the difference between
    // seven and eight waves per SIMD for rows up to 1 KB: 16 batches of 1024 x 1 KB 272 -> 253 us, one
    // batch 33.5 -> 32.7 us.  Four cost 20; four for the first pairs only, or all bytes of a thread's
    // positions requested before the first table read, gained nothing.  Two for the 2 KB forms alone,
    // which have the registers: 8 batches of 32 x 100 kbp 705 -> 730 us; two only in passes in which every
    // thread has two probes, one in the others: 700 -> 715 us.)
    constexpr int kProbes = 1;
    const int wv = (NT == 64) ? 0 : (tid >> 6);
    uint32_t *qn = red + 4 * (NT / 64);        // number of merges queued in the current round
    uint32_t *cn = qn + 1;                     // number of candidates queued in the current round
    uint32_t *capf = qn + 2;                   // walks of the current round that gave up (see kWalkCap)
    // Steps a candidate walks along its left chain before it gives up.  Chains are a few steps
    // long, except inside a run of equal pairs (x x x x ..., every pair has the rank of its left
    // neighbour), where position i would walk i steps.  A candidate that gives up goes onto a list
    // (the far end of the candidate queue).  Up to kLateMax of them (a homopolymer or microsatellite
    // of some dozen copies) then finish their walks, one per thread; with more, the round decides
    // all its candidates again by a scan over the positions instead (below), which costs about as
    // much as a round.
    constexpr int kWalkCap = 24;
    constexpr uint32_t kLateMax = 64;
    // position i belongs to thread i % NT: in every pass the lanes of a wave touch consecutive
    // positions, so the LDS state arrays are read and written without bank conflicts

    PhaseClock clk;
    // a position's product and gate as 16-bit halves of its word of PG
    const uint16_t *const product_of = reinterpret_cast<const uint16_t *>(PG), *const gate_of = product_of + 1;
    // symbols, links and the initial pair of every position, kProbes pairs of table reads in flight at a time
    uint32_t cmin = kEmptyKey, cgate = kEmptyKey;
    D[tid] = 0;
    if (tid == 0) { *qn = 0; *cn = 0; *capf = 0; }
    // With PER > 0 the row's bytes come into LDS first (the candidate queue is free until the first
    // round), 8 aligned bytes per thread: one trip to memory for the whole row instead of one per
    // batch of table reads.  Only a word that reaches over the row's first or last byte is put
    // together from single bytes, so that nothing outside the row is read.
    uint8_t *stage = reinterpret_cast<uint8_t *>(C);
    int head = 0;
    // The single-character ids of a word's eight bytes, stored where the word lies inside
    // [char_lo, char_hi).  The eight ids are requested together whether the word lies wholly inside
    // the range or not (a load, a wait and a store per byte made the two words at the range's ends a
    // chain of eight trips to the cache, for which the whole team waited).
    auto chars_of_word = [&](const int first, const uint2 v, auto id_of) {
        int32_t c[8];
#pragma unroll
        for (int q = 0; q < 8; ++q) c[q] = id_of(((q < 4 ? v.x : v.y) >> (8 * (q & 3))) & 255u);
        if (first >= char_lo && first + 8 <= char_hi) {
            const bpe_int4_a4 x0 = {c[0], c[1], c[2], c[3]}, x1 = {c[4], c[5], c[6], c[7]};
            __builtin_nontemporal_store(x0, reinterpret_cast<bpe_int4_a4 *>(char_ids + first));
            __builtin_nontemporal_store(x1, reinterpret_cast<bpe_int4_a4 *>(char_ids + first + 4));
            if (char_mask) {
                __builtin_nontemporal_store((bpe_u32_a1)0x01010101u, reinterpret_cast<bpe_u32_a1 *>(char_mask + first));
                __builtin_nontemporal_store((bpe_u32_a1)0x01010101u, reinterpret_cast<bpe_u32_a1 *>(char_mask + first + 4));
            }
        } else {
#pragma unroll
            for (int q = 0; q < 8; ++q) {
                const int pos = first + q;
                if (pos >= char_lo && pos < char_hi) {
                    char_ids[pos] = c[q];
                    if (char_mask) char_mask[pos] = 1;
                }
            }
        }
    };
    // Teams of 256 threads (pieces of at least 1 KB: the merge queue holds 1 KB or more and is free
    // until the first round decides) bring the table of the 256 ids into LDS beside the row's
    // bytes, one entry per thread in the same trip to memory, and look the ids up there once the
    // bytes are staged: looked up in memory, the ids were a second trip behind the bytes.
    constexpr bool kIdsFromLds = CHARS && PER > 0 && NT == 256;
    int32_t *const ids_s = reinterpret_cast<int32_t *>(Q);
    if (PER > 0) {
        int32_t id_mine = 0;
        if (kIdsFromLds) id_mine = char_lut[tid];
        head = (int)(reinterpret_cast<uintptr_t>(src) & (uintptr_t)7);
        // (derived from src by pointer arithmetic, so that the loads stay loads from global memory:
        // through an address rebuilt from an integer they become flat loads, which count as LDS
        // accesses too)
        const uint2 *const words = reinterpret_cast<const uint2 *>(src - head);
        const int n_words = (head + n0 + 7) >> 3;
        for (int wd = tid; wd < n_words; wd += NT) {
            const int first = 8 * wd - head;                  // row position of the word's first byte
            uint2 v;
            if (first >= 0 && first + 8 <= n0) {
                v = words[wd];
            } else {
                // (all eight bytes requested together, from positions clamped into the row: a load
                // behind a condition each is a chain of eight trips to the cache, which a row that
                // does not start on an 8-byte boundary pays in its first and its last word while the
                // whole team waits)
                uint32_t b[8];
#pragma unroll
                for (int q = 0; q < 8; ++q) {
                    const int pos = first + q;
                    b[q] = src[pos < 0 ? 0 : (pos < n0 ? pos : n0 - 1)];
                }
                uint32_t lo = 0, hi = 0;
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    if (first + q >= 0 && first + q < n0) lo |= b[q] << (8 * q);
                    if (first + 4 + q >= 0 && first + 4 + q < n0) hi |= b[4 + q] << (8 * q);
                }
                v = uint2{lo, hi};
            }
            *reinterpret_cast<uint2 *>(stage + 8 * wd) = v;
            if (CHARS && !kIdsFromLds && first + 8 > char_lo && first < char_hi)
                chars_of_word(first, v, [&](uint32_t byte) -> int32_t { return char_lut[byte]; });
        }
        if (kIdsFromLds) ids_s[tid] = id_mine;
        team_sync<NT>();
        if (kIdsFromLds) {
            for (int wd = tid; wd < n_words; wd += NT) {
                const int first = 8 * wd - head;
                if (first + 8 > char_lo && first < char_hi)
                    chars_of_word(first, *reinterpret_cast<const uint2 *>(stage + 8 * wd),
                                  [&](uint32_t byte) -> int32_t { return ids_s[byte]; });
            }
        }
    }
    auto byte_at = [&](int i) -> uint32_t { return PER > 0 ? stage[head + i] : src[i]; };
    if (PER > 0 && first) {
        // the first pairs by byte class: one 8-byte read from the workgroup's own table per position
        // (byte_to_sym is not staged then: byte_to_sym_far is the table in memory)
        for (int i = tid; i < n0; i += NT) {
            const uint32_t ba = byte_at(i), bb = i + 1 < n0 ? byte_at(i + 1) : 0u;
            const uint32_t ca = first->cls(ba), cb = i + 1 < n0 ? first->cls(bb) : kNoClass;
            uint2 rule = uint2{kNone, kNone | (kNone << 16)};
            if ((ca | cb) < (uint32_t)kFirstClasses) rule = first->rule[ca * kFirstClasses + cb];
            PosRec<IT> x;
            x.r = (IT)rule.x;
            x.nx = (i + 1 < n0) ? (IT)(i + 1) : NIL;
            x.pv = (i > 0) ? (IT)(i - 1) : NIL;
            // (the class's symbol is read from LDS whatever the class, and the table in memory only
            // behind a branch.  Left to the compiler, the two reads become one flat load from a
            // selected address, which counts as an access to memory: every position then waits for
            // all stores that are still under way.  The empty asm keeps the LDS read where it is.)
            uint32_t sym_a = first->sym[ca & (uint32_t)(kFirstClasses - 1)];
            asm volatile("" : "+v"(sym_a));
            if (ca >= (uint32_t)kFirstClasses) sym_a = byte_to_sym_far[ba];
            x.s = (IT)sym_a;
            P[i] = x;
            PG[i] = rule.y;
            if (rule.x != kNone) { cmin = umin(cmin, rule.x); cgate = umin(cgate, rule.y >> 16); }
        }
    } else
    for (int i0 = tid; i0 < n0; i0 += kProbes * NT) {
        decltype(pair_probe(pt, 0u, 0u)) e[kProbes];
        uint32_t sa[kProbes], sb[kProbes];
#pragma unroll
        for (int j = 0; j < kProbes; ++j) {
            const int i = i0 + j * NT;
            const bool ok = i + 1 < n0;
            sa[j] = i < n0 ? byte_to_sym[byte_at(i)] : 0u;
            sb[j] = ok ? byte_to_sym[byte_at(i + 1)] : 0u;
            e[j] = pair_probe(pt, ok ? sa[j] : 0u, sb[j]);
        }
#pragma unroll
        for (int j = 0; j < kProbes; ++j) {
            const int i = i0 + j * NT;
            if (i >= n0) continue;
            PairInfo pi{kNone, kNoPg};
            if (i + 1 < n0) pi = pair_finish(pt, sa[j], sb[j], e[j]);
            PosRec<IT> x;
            x.r = (IT)pi.rank;
            x.nx = (i + 1 < n0) ? (IT)(i + 1) : NIL;
            x.pv = (i > 0) ? (IT)(i - 1) : NIL;
            x.s = (IT)sa[j];
            P[i] = x;
            PG[i] = pi.pg;
            if (pi.rank != kNone) { cmin = umin(cmin, pi.rank); cgate = umin(cgate, pi.pg >> 16); }
        }
    }

    // ranks of the thread's own positions (position tid + k * NT is its k-th), kept up to date by
    // the refresh at the end of every round: the candidates of a round are then found without
    // reading LDS
    uint32_t myr[PER > 0 ? PER : 1];
    if (PER > 0) {
#pragma unroll
        for (int k = 0; k < PER; ++k) {
            const int i = tid + k * NT;
            myr[k] = i < n0 ? (uint32_t)P[i].r : kNone;      // written by this thread just above
        }
    }

    clk.lap(kPhInitial);
    int flip = 0;
    int budget = n0 + 8;                       // every round merges at least one pair
    bool stuck = false;
    for (;;) {
        if (--budget < 0) { stuck = true; break; }   // cannot happen; keeps the loop bounded
        uint32_t rmin, gate;
        if (sizeof(IT) == 2) team_min2_u16<NT>(cmin, cgate, red + flip * (NT / 64) * 2, wv, rmin, gate);   // (syncs the team)
        else team_min2<NT>(cmin, cgate, red + flip * (NT / 64) * 2, wv, rmin, gate);
        flip ^= 1;
        clk.lap(kPhMinimum);
        if (rmin >= kNone) break;
        clk.count(kPhRounds, 1);
        const bool single = gate <= rmin;          // non-monotone table: one merge this round
        uint32_t leftmost = 0;
        if (single) {
            uint32_t mypos = kEmptyKey;
            if (cmin == rmin)
                for (int i = tid; i < n0; i += NT)
                    if (P[i].r == rmin) { mypos = (uint32_t)i; break; }
            uint32_t dummy;
            if (sizeof(IT) == 2) team_min2_u16<NT>(mypos, mypos, red + flip * (NT / 64) * 2, wv, leftmost, dummy);
            else team_min2<NT>(mypos, mypos, red + flip * (NT / 64) * 2, wv, leftmost, dummy);
            flip ^= 1;
        }
        const uint32_t limit = single ? rmin + 1 : gate;

        // decide (reads only); a pair that merges is put on the round's queue.  The candidates
        // (pairs with a rank below the limit, typically a quarter of the live positions, spread
        // unevenly over the threads) are first collected on a queue of their own and then dealt out
        // one per thread: every thread walks one candidate's chains at a time, with all lanes of a
        // wave busy, instead of its own positions one after the other with most lanes idle.
        int ncand = 0;
        if (single) {
            if (tid == 0) { Q[0] = (IT)leftmost; *qn = 1; }
        } else {
            const int lane = tid & 63;
            if (PER > 0) {
                // ranks from registers, one ballot per position of the thread, one queue atomic
                // per wave and round
                uint64_t bal[PER > 0 ? PER : 1];
                uint32_t total = 0;
#pragma unroll
                for (int k = 0; k < PER; ++k) {
                    bal[k] = __ballot(myr[k] < limit);    // (kNone beyond the row's end: never below)
                    total += (uint32_t)__builtin_popcountll(bal[k]);
                }
                if (total != 0) {                         // (uniform over the wave)
                    uint32_t at = 0;
                    if (lane == 0) at = atomicAdd(cn, total);
                    at = (uint32_t)__builtin_amdgcn_readfirstlane((int)at);
#pragma unroll
                    for (int k = 0; k < PER; ++k) {
                        if (myr[k] < limit)                       // (the lane's own bit of the ballot)
                            C[at + lanes_below(bal[k])] =
                                (IT)(tid + k * NT);
                        at += (uint32_t)__builtin_popcountll(bal[k]);
                    }
                }
            } else {
                for (int b0 = 0; b0 < n0; b0 += 4 * NT) {     // the same trip count for every lane
                    uint64_t bal[4];
                    uint32_t total = 0;
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        const int i = b0 + k * NT + tid;
                        bal[k] = __ballot(cmin < limit && i < n0 && (uint32_t)P[i].r < limit);
                        total += (uint32_t)__builtin_popcountll(bal[k]);
                    }
                    if (total == 0) continue;                 // (uniform over the wave)
                    uint32_t at = 0;
                    if (lane == 0) at = atomicAdd(cn, total);
                    at = (uint32_t)__builtin_amdgcn_readfirstlane((int)at);
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        if (bal[k] >> lane & 1ull)
                            C[at + lanes_below(bal[k])] =
                                (IT)(b0 + k * NT + tid);
                        at += (uint32_t)__builtin_popcountll(bal[k]);
                    }
                }
            }
            team_sync<NT>();
            clk.lap(kPhCollect);
            ncand = (int)*cn;
            for (int c0 = 0; c0 < ncand; c0 += NT) {      // the same trip count for every lane
                const int c = c0 + tid;
                bool merges = false;
                int i = 0;
                if (c < ncand) {
                    i = (int)C[c];
                    const PosRec<IT> x = P[i];
                    const uint32_t r = x.r;
                    // both neighbours' records are requested together
                    PosRec<IT> yl = P[x.pv != NIL ? x.pv : (IT)i];
                    PosRec<IT> yr = P[x.nx != NIL ? x.nx : (IT)i];
                    uint32_t chain = 0, rp = r;
                    IT q = x.pv;
                    bool gave_up = false;
                    while (q != NIL && yl.r <= rp) {      // candidates to the left with key <= ours
                        if (chain == (uint32_t)kWalkCap) { gave_up = true; break; }
                        ++chain; rp = yl.r; q = yl.pv;
                        if (q != NIL) yl = P[q];
                    }
                    uint32_t chain_r = 0;
                    rp = r; q = x.nx;
                    while (q != NIL && yr.r < rp) {       // candidates to the right with key < ours
                        ++chain_r; rp = yr.r; q = yr.nx;
                        if (q != NIL) yr = P[q];
                    }
                    merges = !gave_up && ((chain | chain_r) & 1u) == 0;
                    if (gave_up) {
                        const uint32_t k = atomicAdd(capf, 1u);
                        if (k < kLateMax && n0 - 1 - (int)k >= ncand) C[n0 - 1 - (int)k] = (IT)i;
                    }
                }
                // one queue atomic per wave (64 atomics on one LDS word take their turns)
                const uint64_t bal = __ballot(merges);
                if (bal != 0) {                           // (uniform over the wave)
                    uint32_t at = 0;
                    if (lane == 0) at = atomicAdd(qn, (uint32_t)__builtin_popcountll(bal));
                    at = (uint32_t)__builtin_amdgcn_readfirstlane((int)at);
                    if (merges) Q[at + lanes_below(bal)] = (IT)i;
                }
            }
        }
        team_sync<NT>();
        clk.lap(kPhDecide);
        const uint32_t late = single ? 0u : *capf;
        const bool by_scan = late > kLateMax || ncand + (int)late > n0;
        if (late != 0 && !by_scan) {
            // the few walks that gave up, in full, one per thread
            const int lane = tid & 63;
            bool merges = false;
            int i = 0;
            if ((uint32_t)tid < late) {
                i = (int)C[n0 - 1 - tid];
                const PosRec<IT> x = P[i];
                uint32_t chain = 0, rp = x.r;
                IT q = x.pv;
                PosRec<IT> y = P[q != NIL ? q : (IT)i];
                while (q != NIL && y.r <= rp) {
                    ++chain; rp = y.r; q = y.pv;
                    if (q != NIL) y = P[q];
                }
                uint32_t chain_r = 0;
                rp = x.r; q = x.nx;
                y = P[q != NIL ? q : (IT)i];
                while (q != NIL && y.r < rp) {
                    ++chain_r; rp = y.r; q = y.nx;
                    if (q != NIL) y = P[q];
                }
                merges = ((chain | chain_r) & 1u) == 0;
            }
            const uint64_t bal = __ballot(merges);
            if (bal != 0) {                               // (uniform over the wave)
                uint32_t at = 0;
                if (lane == 0) at = atomicAdd(qn, (uint32_t)__builtin_popcountll(bal));
                at = (uint32_t)__builtin_amdgcn_readfirstlane((int)at);
                if (merges) Q[at + lanes_below(bal)] = (IT)i;
            }
            team_sync<NT>();
        }
        if (late != 0 && by_scan) {
            // Exact decision for every candidate of the round without walking to the left.  The
            // left chain of candidate i has even length iff x(i) = 0, where x runs over the live
            // positions from left to right: x(i) = x(left neighbour) ^ 1 if that neighbour is a
            // candidate with a rank <= ours, else 0.  Every position is a function on that one
            // bit (keep: a dead position; flip; set to 0), functions compose, so the positions
            // are taken NT at a time in index order (which is the list's order), a wave at a time
            // from two ballots, with the bit carried from wave to wave and from block to block.
            constexpr int NW = NT / 64;
            const int lane = tid & 63;
            team_sync<NT>();                            // everyone has read the count
            if (tid == 0) *qn = 0;
            team_sync<NT>();
            uint32_t carry = 0;                         // x of the last live position before the block
            int blk = 0;
            for (int b0 = 0; b0 < n0; b0 += NT, blk ^= 1) {      // the same trip count for every lane
                const int i = b0 + tid;
                bool keep = true, flips = false, cand = false;
                PosRec<IT> x;
                x.r = DEAD; x.nx = NIL; x.pv = NIL; x.s = DEAD;
                if (i < n0) x = P[i];
                if (x.s != DEAD) {
                    cand = (uint32_t)x.r < limit;
                    bool link = false;
                    if (cand && x.pv != NIL) link = (uint32_t)P[x.pv].r <= (uint32_t)x.r;
                    keep = link; flips = link;
                }
                const uint64_t kp = __ballot(keep), fl = __ballot(flips);
                const uint64_t upto = lane == 63 ? ~0ull : ((2ull << lane) - 1ull);     // lanes 0 .. lane
                const uint64_t resets = ~kp & upto;
                uint64_t seg = upto;
                if (resets != 0) seg &= ~((1ull << (63 - __builtin_clzll(resets))) - 1ull);    // from the last reset on
                uint32_t xi = (uint32_t)__builtin_popcountll(fl & seg) & 1u;              // with 0 coming in
                const bool w_keep = kp == ~0ull;
                const uint32_t w_bit = (uint32_t)__builtin_amdgcn_readlane((int)xi, 63);
                uint32_t into_wave = carry;
                if (NW > 1) {
                    if (lane == 0) red[blk * NW + wv] = (w_keep ? 2u : 0u) | w_bit;
                    team_sync<NT>();
                    uint32_t c = carry;
#pragma unroll
                    for (int w = 0; w < NW; ++w) {
                        if (w == wv) into_wave = c;
                        const uint32_t e = red[blk * NW + w];
                        c = (e & 2u) ? (c ^ (e & 1u)) : (e & 1u);
                    }
                    carry = c;
                } else {
                    carry = w_keep ? (carry ^ w_bit) : w_bit;
                }
                if (resets == 0) xi ^= into_wave;
                bool merges = false;
                if (cand && xi == 0) {
                    uint32_t chain_r = 0, rp = x.r;
                    IT q = x.nx;
                    PosRec<IT> yr = P[q != NIL ? q : (IT)i];
                    while (q != NIL && yr.r < rp) {       // candidates to the right with key < ours
                        ++chain_r; rp = yr.r; q = yr.nx;
                        if (q != NIL) yr = P[q];
                    }
                    merges = (chain_r & 1u) == 0;
                }
                const uint64_t bal = __ballot(merges);
                if (bal != 0) {                           // (uniform over the wave)
                    uint32_t at = 0;
                    if (lane == 0) at = atomicAdd(qn, (uint32_t)__builtin_popcountll(bal));
                    at = (uint32_t)__builtin_amdgcn_readfirstlane((int)at);
                    if (merges) Q[at + lanes_below(bal)] = (IT)i;
                }
            }
            team_sync<NT>();
        }
        const int nm = (int)*qn;                   // merges of this round (they do not overlap)
        clk.lap(kPhLate);
        clk.count(kPhMerges, nm);

        // apply: position i absorbs its right neighbour j; one merge per thread and pass
        for (int m = tid; m < nm; m += NT) {
            const IT i = Q[m];
            const IT j = P[i].nx;
            const IT k = P[j].nx;
            P[i].s = (IT)product_of[2 * (int)i];
            P[i].nx = k;
            P[j].s = DEAD;
            P[j].r = DEAD;
            if (k != NIL) P[k].pv = i;
            D[(int)(j % NT)] = 1;             // j's owner must refresh its cached minimum
        }
        team_sync<NT>();
        clk.lap(kPhApply);

        // re-rank the two pairs around every new symbol: probe m is the pair (new, right
        // neighbour), probe nm + m the pair (left neighbour, new).  The probes are dealt evenly to
        // the threads, kProbes pairs of table reads in flight per thread.
        for (int p0 = tid; p0 < 2 * nm; p0 += kProbes * NT) {
            decltype(pair_probe(pt, 0u, 0u)) e[kProbes];
            uint32_t sa[kProbes], sb[kProbes];
            IT target[kProbes];
            bool valid[kProbes];
#pragma unroll
            for (int j = 0; j < kProbes; ++j) {
                const int p = p0 + j * NT;
                sa[j] = 0; sb[j] = 0; target[j] = NIL; valid[j] = false;
                if (p < 2 * nm) {
                    // (probes 0 .. nm - 1 are the pairs to the right, nm .. 2 nm - 1 those to the left:
                    // with the two kinds alternating lane by lane every wave ran both branches)
                    const bool to_the_left = p >= nm;
                    const IT i = Q[to_the_left ? p - nm : p];
                    const PosRec<IT> x = P[i];
                    if (to_the_left) {
                        target[j] = x.pv;
                        if (x.pv != NIL) { sa[j] = P[x.pv].s; sb[j] = x.s; valid[j] = true; }
                    } else {
                        target[j] = i;
                        if (x.nx != NIL) { sa[j] = x.s; sb[j] = P[x.nx].s; valid[j] = true; }
                    }
                }
                e[j] = pair_probe(pt, sa[j], sb[j]);
            }
#pragma unroll
            for (int j = 0; j < kProbes; ++j) {
                if (target[j] == NIL) continue;       // no probe, or no left neighbour
                PairInfo pi{kNone, kNoPg};
                if (valid[j]) pi = pair_finish(pt, sa[j], sb[j], e[j]);
                const int q = (int)target[j];
                P[q].r = (IT)pi.rank; PG[q] = pi.pg;
                D[q % NT] = 1;
            }
        }
        team_sync<NT>();
        clk.lap(kPhRerank);
        if (tid == 0) { *qn = 0; *cn = 0; *capf = 0; }   // seen by the next round's decide (a sync lies between)

        if (D[tid]) {
            D[tid] = 0;
            cmin = kEmptyKey; cgate = kEmptyKey;
            if (PER > 0) {
#pragma unroll
                for (int k = 0; k < PER; ++k) {
                    const int i = tid + k * NT;
                    const uint32_t r = i < n0 ? (uint32_t)P[i].r : kNone;
                    const uint32_t g = gate_of[2 * (i < n0 ? i : tid)];      // read beside the rank, not after it
                    myr[k] = r;
                    if (r != kNone) { cmin = umin(cmin, r); cgate = umin(cgate, g); }
                }
            } else {
                for (int i = tid; i < n0; i += NT) {
                    const uint32_t r = P[i].r;
                    if (r != kNone) { cmin = umin(cmin, r); cgate = umin(cgate, gate_of[2 * i]); }
                }
            }
        }
        clk.lap(kPhRefresh);
    }
    clk.count(kPhPositions, n0);
    clk.count(kPhItems, 1);

    if (raw_out) {
        // chunk of a long row: hand back the symbol at every start position (kNone elsewhere) and
        // the number of tokens that start in [mid_lo, mid_hi), the stretch no neighbouring chunk
        // shares; the seam and gather kernels assemble the row
        uint32_t live = 0;
        for (int i = tid; i < n0; i += NT) {
            const uint16_t sy = stuck ? (uint16_t)kNone : (uint16_t)P[i].s;
            raw_out[i] = sy;
            live += (i >= mid_lo && i < mid_hi && sy != (uint16_t)kNone) ? 1u : 0u;
        }
        uint32_t total;
        team_sync<NT>();                         // red may still be read by the last round's minimum
        (void)team_exclusive_sum<NT>(live, red, wv, total);
        if (tid == 0) *mid_out = (int32_t)total;
        clk.lap(kPhOutput);
        clk.flush(tid);
        return 0;
    }
    // Compact the live symbols to the output, in position order.  Position i = pass * NT + tid, so a
    // pass is NT consecutive positions: a ballot per wave gives every lane its place among the
    // wave's live symbols, the waves' counts of a block of passes go through LDS (PG is free by
    // now: every thread left the loop behind the same barrier), and the stores of a wave go to
    // consecutive cells.  (A contiguous piece per thread, as before, cost a fifth of a 1 KB row's
    // time: strided LDS reads, two scans and stores scattered over the row.)
    constexpr int NW = NT / 64;
    // (a row of at most PER passes never has more in a block: the passes beyond cost registers for nothing)
    constexpr int kBlockPasses = (PER > 0 && PER < 8) ? PER : 8;
    uint32_t *wave_cnt = PG;                                         // [kBlockPasses][NW]
    const int lane = tid & 63;
    uint32_t done = 0;                                               // tokens of earlier blocks of passes
    // PAD: where row pad_row of the padded output lies and what pads it, from the kernel's
    // arguments (the first of them is the BpeArgs), read here and not before the merges
    int pad_stride = 0, pad_elem = 4, pad_left = 0;
    int32_t pad_id = 0;
    uint8_t *pad_mask = nullptr;
    const int32_t *remap2 = nullptr;
    if (PAD) {
        const BpeArgsInMemory ka = kernel_args_now();
        pad_stride = (int)ka->pad_stride; pad_elem = ka->pad_elem; pad_left = ka->pad_left; pad_id = ka->pad_id;
        remap2 = ka->pad_remap;
        out = reinterpret_cast<int32_t *>(reinterpret_cast<char *>(ka->pad_ids) +
                                          (int64_t)pad_row * ka->pad_stride * pad_elem);
        if (ka->pad_mask) pad_mask = ka->pad_mask + (int64_t)pad_row * ka->pad_stride;
    }
    // cell c of a padded row, in the row's own integer width
    auto put_cell = [&](int c, int32_t v) {
        if (!PAD || pad_elem == 4) out[c] = v;
        else if (pad_elem == 8) reinterpret_cast<int64_t *>(out)[c] = (int64_t)v;
        else if (pad_elem == 2) reinterpret_cast<int16_t *>(out)[c] = (int16_t)v;
        else reinterpret_cast<uint8_t *>(out)[c] = (uint8_t)v;
    };
    // padding on the left: the row's tokens end at its last cell, so their number comes first
    int shift = 0;
    if (PAD && pad_left) {
        uint32_t mine = 0, total;
        for (int i = tid; i < n0; i += NT) mine += (uint32_t)(P[i].s != DEAD);
        (void)team_exclusive_sum<NT>(mine, red, wv, total);
        shift = pad_stride - (int)(total < (uint32_t)pad_stride ? total : (uint32_t)pad_stride);
    }
    for (int i0 = 0; i0 < n0; i0 += kBlockPasses * NT) {
        uint32_t sy[kBlockPasses], before[kBlockPasses];
        int32_t id[kBlockPasses];
#pragma unroll
        for (int k = 0; k < kBlockPasses; ++k) {
            const int i = i0 + k * NT + tid;
            sy[k] = i < n0 ? (uint32_t)P[i].s : kNone;
        }
        // the ids of all symbols of the block are requested before the first of them is stored (a
        // load behind a store waits for the store as well: one trip to the cache per pass otherwise)
#pragma unroll
        for (int k = 0; k < kBlockPasses; ++k)
            id[k] = (sy[k] != kNone && out_remap) ? out_remap[sy[k]] : (int32_t)sy[k];
#pragma unroll
        for (int k = 0; k < kBlockPasses; ++k) {
            const uint64_t live = __ballot(sy[k] != kNone);
            before[k] = lanes_below(live);
            if (lane == 0) wave_cnt[k * NW + wv] = (uint32_t)__builtin_popcountll(live);
        }
        if (PAD && remap2) {
#pragma unroll
            for (int k = 0; k < kBlockPasses; ++k)
                if (sy[k] != kNone) id[k] = remap2[id[k]];
        }
        team_sync<NT>();
        uint32_t at = done;
#pragma unroll
        for (int k = 0; k < kBlockPasses; ++k) {
            uint32_t mine = at;
#pragma unroll
            for (int w = 0; w < NW; ++w) {
                const uint32_t c = wave_cnt[k * NW + w];
                if (w < wv) mine += c;
                at += c;
            }
            const uint32_t cell = mine + before[k];
            if (sy[k] != kNone && (!PAD || cell < (uint32_t)pad_stride)) put_cell(shift + (int)cell, id[k]);
        }
        done = at;
        team_sync<NT>();                                             // wave_cnt is rewritten by the next block
    }
    if (tid == 0) *out_len = stuck ? -2 : (int32_t)done;
    if (PAD) {
        const int kept = (int)done < pad_stride ? (int)done : pad_stride;
        const int pad_from = pad_left ? 0 : kept, pad_to = pad_left ? pad_stride - kept : pad_stride;
        for (int i = pad_from + tid; i < pad_to; i += NT) put_cell(i, pad_id);
        if (pad_mask)
            for (int i = tid; i < pad_stride; i += NT) pad_mask[i] = (i >= pad_from && i < pad_to) ? 0 : 1;
    }
    clk.lap(kPhOutput);
    clk.flush(tid);
    return (int32_t)done;
}

// ---- long rows in chunks -------------------------------------------------------------------
//
// A row longer than one extended chunk is cut into chunks of kChunkCore bytes, each extended by
// kChunkOverlap bytes on both sides, and every extended chunk is merged on its own.  Two
// neighbouring chunks A and B are then joined at a seam: a position p inside their overlap
// where both runs end with a token boundary, the token ending at p is the same token in both,
// and the token starting at p is the same token in both.  A token's own merge history depends
// only on its string, so at such a p the two boundary symbols evolve identically in A and B;
// taking A's merges left of p and B's merges right of p therefore is a legal run of the
// (rank, position) order on the whole row, hence THE run (with a merge table in which every
// rule's product is only used by higher-ranked rules, so that merges happen in key order).
// If an overlap holds no such p (e.g. a tandem repeat longer than the overlap), the row is
// redone by the whole-row kernel.
constexpr int kLdsCap = 4096;            // longest piece any LDS kernel variant takes
// 2048-byte extended chunks: 31 KB of LDS state, five workgroups per CU; measured faster than
// 4096-byte chunks (fewer positions per thread, more chunks in flight) and than 1408- or 1536-byte
// ones (the overlap is work done twice: its share of a chunk decides).  Overlap: with 64 bytes 0.3 %
// of the seams of the 32000-vocabulary benchmark rows (10 % tandem repeats of up to 180 bp) find no
// position, with 96 none of 5,088, with 128 none of 35,200 (CPU count with the oracle).
constexpr int kChunkOverlap = 128;
constexpr int kChunkCore = 2048 - 2 * kChunkOverlap;
constexpr int kLongThreads = 1024;
constexpr int kLongGrid = 64;            // slabs of scratch for the whole-row fallback kernel

// The work list: the chunks of all chunked rows first (the largest items), then the rows that are
// one item each, in classes of falling length.  Items are handed out in that order, so the last
// ones to start are short: with rows in their given order a 2 KB item that starts last leaves most
// teams idle for its whole duration (ragged benchmark batch: 0.299 -> 0.289 ms).
constexpr int kSingleClasses = 3;

// The items beyond one per team are handed out through kDealers counters instead of one: an
// atomic on one address takes its turn behind all others (about 12 ns each), which for 100,000
// short rows is longer than their merging.  Counter c hands out the items whose number is c modulo
// kDealers, to the teams whose number is c modulo kDealers: every counter's share of the list,
// which runs from large items to small ones, looks like the whole.
constexpr int kDealers = 16;
constexpr int kDealerStride = 64;         // int32 words between two counters (256 bytes)

struct BpePlan {                          // device arrays inside the scratch buffer
    int32_t *counts;      // [0] items, [1] chunk items, [3] failed rows, [4 + c] single rows of class c
    int32_t *deal;        // [2][kDealers * kDealerStride] the work counters (second bank: a launch for the shortest rows alone)
    int32_t *mc_off;      // [n_rows + 1] first chunk slot of a row (multi-chunk rows only)
    int4 *rec;           // [max_mc] a chunk item: {row, chunk of the row, chunks of the row, row length}
    int32_t *single[kSingleClasses];   // [n_rows] each: the rows that are one item, longest class first
    int32_t *seam;        // [max_mc] seam to the right of a chunk (row position), -1 = none found
    int32_t *cnt;         // [max_mc][4] tokens of a chunk: in the stretch it shares with no other chunk, from the
                          // seam on its left to that stretch, from that stretch to the seam on its right
    int32_t *row_fail;    // [n_rows] 1 = redo the row with the whole-row kernel
    int32_t *tile_sums;   // [n_rows / 4096 + 1][8] what the rows of a tile add to the work list's scans, and its failed rows
    uint16_t *chunk_sym;  // [max_mc][ext]
    uint8_t *slabs;       // whole-row fallback state
    size_t slab_bytes, total_bytes;
    int64_t max_items, max_mc;
    int core, overlap, ext;   // chunk core, overlap on each side, core + 2 * overlap
    int n_slabs;              // workgroups of the whole-row fallback kernel (one slab of state each)
};

static size_t long_slab_bytes(int64_t max_len)
{
    const size_t n = ((size_t)max_len + 7) & ~(size_t)7;
    return ((n * 26) + 255) & ~(size_t)255;     // 16 (records) + 2 + 2 (product, gate) + 2 + 4 (queues)
}

// Chunk geometry of a table's calls.  The shipped values are the constants above;
// dnatok_bpe_table_set_chunk_geometry lets a test run the chunk / seam / fallback machinery with
// chunks so small that every few hundred bytes of a row hold a seam.

// A batch whose long rows make far fewer chunks than teams fit the chip (a few rows of a few
// thousand bytes each) is cut finer, down to a core of 512 bytes: more, shorter items run side by
// side, and the batch is latency-bound either way (one row of 100 kbp: 48 -> 38 us per call).
// Only with the shipped geometry, and only when the batch has long rows at all.
static void chunk_geometry(const dnatok_bpe_t *t, int *core, int *overlap, int64_t max_len, int64_t total)
{
    *core = t ? t->chunk_core.load(std::memory_order_relaxed) : 0;
    *overlap = t ? t->chunk_overlap.load(std::memory_order_relaxed) : 0;
    if (*core == 0 || *overlap == 0) { *core = kChunkCore; *overlap = kChunkOverlap; }
    if (*core == kChunkCore && *overlap == kChunkOverlap && max_len > kChunkCore + 2 * kChunkOverlap) {
        constexpr int64_t kTeams = 1024;                 // about what is resident at once
        int64_t c = (total / kTeams + 127) & ~(int64_t)127;
        if (c < 512) c = 512;
        if (c < kChunkCore) *core = (int)c;
    }
}

static BpePlan make_plan(const dnatok_bpe_t *t, uint8_t *base, int64_t n_rows, int64_t max_len, int64_t total,
                         int64_t max_slabs = kLongGrid)
{
    BpePlan p{};
    chunk_geometry(t, &p.core, &p.overlap, max_len, total);
    p.ext = p.core + 2 * p.overlap;
    auto up = [](size_t v) { return (v + 255) & ~(size_t)255; };
    const bool chunks = max_len > p.ext;
    p.max_items = n_rows + (chunks ? total / p.core + 1 : 0);
    // chunk slots: a chunked row of len bytes takes ceil(len / core) <= len / core + 1 of them, and
    // there are fewer chunked rows than rows, and than total / core (each is longer than a chunk)
    const int64_t by_rows = total / p.core + n_rows + 1, by_bytes = 2 * (total / p.core) + 2;
    p.max_mc = chunks ? (by_rows < by_bytes ? by_rows : by_bytes) : 0;
    size_t o = 0;
    auto take = [&](size_t bytes) { size_t at = o; o = up(o + bytes); return at; };
    const size_t o_counts = take(64);
    const size_t o_deal = take(2 * 4 * (size_t)kDealers * kDealerStride);
    const size_t o_mc_off = take(4 * (size_t)(n_rows + 1));
    const size_t o_rec = take(16 * (size_t)p.max_mc);
    size_t o_single[kSingleClasses];
    for (int c = 0; c < kSingleClasses; ++c) o_single[c] = take(4 * (size_t)n_rows);
    const size_t o_seam = take(4 * (size_t)p.max_mc);
    const size_t o_cnt = take(16 * (size_t)p.max_mc);
    const size_t o_fail = take(4 * (size_t)n_rows);
    const size_t o_tiles = take(4 * 8 * (size_t)(n_rows / 4096 + 1));
    const size_t o_sym = take(2 * (size_t)p.ext * (size_t)p.max_mc);
    p.slab_bytes = chunks ? long_slab_bytes(max_len) : 0;
    const int64_t slabs = n_rows < max_slabs ? n_rows : max_slabs;
    p.n_slabs = (int)(slabs < 1 ? 1 : slabs);
    const size_t o_slabs = take(chunks ? p.slab_bytes * (size_t)p.n_slabs : 0);
    p.total_bytes = o + 256;
    if (base) {
        p.counts = (int32_t *)(base + o_counts);
        p.deal = (int32_t *)(base + o_deal);
        p.mc_off = (int32_t *)(base + o_mc_off);
        p.rec = (int4 *)(base + o_rec);
        for (int c = 0; c < kSingleClasses; ++c) p.single[c] = (int32_t *)(base + o_single[c]);
        p.seam = (int32_t *)(base + o_seam);
        p.cnt = (int32_t *)(base + o_cnt);
        p.row_fail = (int32_t *)(base + o_fail);
        p.tile_sums = (int32_t *)(base + o_tiles);
        p.chunk_sym = (uint16_t *)(base + o_sym);
        p.slabs = base + o_slabs;
    }
    return p;
}

// Work list: ceil(len / core) chunk slots per long row, one entry in its length class per other
// row.  A thread takes four consecutive rows per step, so that a tile of 4096 rows is one round of
// loads and one scan (the kernel is a chain of load latencies and barriers, not work).
// PASS 0: the whole list by one workgroup, tile after tile (up to kPlanTiledFrom rows: one launch).
// More rows take two launches with a workgroup per tile (32,768 rows: 38 us by one workgroup, while
// nothing else runs, against about 10 us for the two): PASS 1 adds up what each tile contributes (and marks the
// rows left to the whole-row kernel), PASS 2 places every tile behind the tiles before it; its
// last workgroup, which sees all the sums, writes the counters.
constexpr int kPlanRows = 4;
constexpr int kPlanTile = 1024 * kPlanRows;
constexpr int64_t kPlanTiledFrom = 2 * kPlanTile + 1;
constexpr int kPlanScans = 1 + kSingleClasses;
constexpr int kPlanInlineRows = 4096;      // the plan kernel writes the chunk entries itself up to this
constexpr int kPlanInlineChunks = 8192;    // many rows and this many chunks (a bound known on the host)

template <int PASS>
__global__ __launch_bounds__(1024) void bpe_plan_kernel(
    const int64_t *__restrict__ offsets, int64_t n_rows, int chunking, int expand_here, BpePlan p)
{
    __shared__ uint32_t wt[kPlanScans + 1][16];
    __shared__ int32_t carry[kPlanScans];
    __shared__ int32_t fail_s;
    __shared__ int32_t s_mc[PASS == 0 ? kPlanInlineRows : 1], s_len[PASS == 0 ? kPlanInlineRows : 1];   // first chunk and length of every row (expand_here)
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    if (threadIdx.x < kPlanScans) carry[threadIdx.x] = 0;
    if (threadIdx.x == 0) fail_s = 0;
    __syncthreads();
    if (PASS == 2) {
        // what the tiles before this one add up to (the last workgroup: all but its own), and their failed rows
        int32_t part[kPlanScans + 1];
#pragma unroll
        for (int q = 0; q <= kPlanScans; ++q) part[q] = 0;
        for (int64_t t = threadIdx.x; t < (int64_t)blockIdx.x; t += 1024)
#pragma unroll
            for (int q = 0; q <= kPlanScans; ++q) part[q] += p.tile_sums[8 * t + q];
#pragma unroll
        for (int q = 0; q <= kPlanScans; ++q) {
            const uint32_t inc = wave_inclusive_sum_u32((uint32_t)part[q]);
            if (lane == 63) wt[q][wv] = inc;
        }
        __syncthreads();
        if (threadIdx.x <= kPlanScans) {
            uint32_t t = 0;
            for (int w = 0; w < 16; ++w) t += wt[threadIdx.x][w];
            if (threadIdx.x < kPlanScans) carry[threadIdx.x] = (int32_t)t; else fail_s = (int32_t)t;
        }
        __syncthreads();
    }
    int32_t n_fail = 0;
    const int64_t first_row = PASS == 0 ? 0 : (int64_t)blockIdx.x * kPlanTile;
    const int64_t end_row = PASS == 0 ? n_rows : (first_row + kPlanTile < n_rows ? first_row + kPlanTile : n_rows);
    for (int64_t base = first_row; base < end_row; base += kPlanTile) {
        const int64_t row0 = base + (int64_t)threadIdx.x * kPlanRows;
        int64_t off[kPlanRows + 1];
#pragma unroll
        for (int r = 0; r <= kPlanRows; ++r) off[r] = row0 + r <= n_rows ? offsets[row0 + r] : 0;
        // what a row adds to each scan: [0] chunk slots, [1 + c] one if it is a single row of class c
        uint32_t add[kPlanRows][kPlanScans], sum[kPlanScans];
#pragma unroll
        for (int q = 0; q < kPlanScans; ++q) sum[q] = 0;
#pragma unroll
        for (int r = 0; r < kPlanRows; ++r) {
#pragma unroll
            for (int q = 0; q < kPlanScans; ++q) add[r][q] = 0;
            if (row0 + r < n_rows) {
                const int64_t len = off[r + 1] - off[r];
                if (len > p.ext && chunking) {
                    add[r][0] = (uint32_t)((len + p.core - 1) / p.core);
                } else {
                    const int c = len > p.ext / 2 ? 0 : (len > p.ext / 4 ? 1 : 2);
#pragma unroll
                    for (int q = 0; q < kSingleClasses; ++q) add[r][1 + q] = q == c ? 1u : 0u;
                }
                const int fail = (len > p.ext && !chunking) ? 1 : 0;
                if (PASS != 2) { p.row_fail[row0 + r] = fail; n_fail += fail; }
            }
#pragma unroll
            for (int q = 0; q < kPlanScans; ++q) sum[q] += add[r][q];
        }
        uint32_t inc[kPlanScans];
#pragma unroll
        for (int q = 0; q < kPlanScans; ++q) {
            inc[q] = wave_inclusive_sum_u32(sum[q]);
            if (lane == 63) wt[q][wv] = inc[q];
        }
        __syncthreads();
        int32_t at[kPlanScans], tot[kPlanScans];
#pragma unroll
        for (int q = 0; q < kPlanScans; ++q) {
            uint32_t b = 0, t = 0;
#pragma unroll
            for (int w = 0; w < 16; ++w) {
                if (w < wv) b += wt[q][w];
                t += wt[q][w];
            }
            at[q] = carry[q] + (int32_t)(b + inc[q] - sum[q]);
            tot[q] = carry[q] + (int32_t)t;
        }
        if (PASS == 1) {                                 // (one tile: the sums are all this pass is for)
            if (threadIdx.x < kPlanScans)
#pragma unroll
                for (int q = 0; q < kPlanScans; ++q) if ((int)threadIdx.x == q) p.tile_sums[8 * (size_t)blockIdx.x + q] = tot[q];
            break;
        }
#pragma unroll
        for (int r = 0; r < kPlanRows; ++r) {
            if (row0 + r >= n_rows) continue;
            const int32_t row = (int32_t)(row0 + r);
            p.mc_off[row] = at[0];
            // the entries of the chunks are written by bpe_expand_kernel (a single workgroup
            // writing tens of thousands of scattered words is bound by its one CU's store path),
            // except for a batch of few chunks, whose entries are written below (a launch less)
            if (PASS == 0 && expand_here) { s_mc[row] = at[0]; s_len[row] = (int32_t)(off[r + 1] - off[r]); }
#pragma unroll
            for (int q = 0; q < kSingleClasses; ++q)
                if (add[r][1 + q]) p.single[q][at[1 + q]] = row;
#pragma unroll
            for (int q = 0; q < kPlanScans; ++q) at[q] += (int32_t)add[r][q];
        }
        __syncthreads();
        if (threadIdx.x < kPlanScans) {
#pragma unroll
            for (int q = 0; q < kPlanScans; ++q) if ((int)threadIdx.x == q) carry[q] = tot[q];
        }
        __syncthreads();
    }
    if (n_fail) atomicAdd(&fail_s, n_fail);
    __syncthreads();
    if (PASS == 1) {
        if (threadIdx.x == 0) p.tile_sums[8 * (size_t)blockIdx.x + kPlanScans] = fail_s;
        return;
    }
    if (PASS == 2) {
        if (blockIdx.x + 1 != gridDim.x) return;         // the last tile's workgroup has the totals
        if (threadIdx.x == 0) fail_s += p.tile_sums[8 * (size_t)blockIdx.x + kPlanScans];
        __syncthreads();
    }
    if (PASS == 0 && expand_here) {
        // chunk c belongs to the last row whose first chunk is at or before c
        const int32_t total = carry[0];
        for (int32_t c = threadIdx.x; c < total; c += 1024) {
            int32_t lo = 0, hi = (int32_t)n_rows;             // first row whose first chunk lies beyond c
            while (lo < hi) {
                const int32_t mid = (lo + hi) >> 1;
                if (s_mc[mid] <= c) lo = mid + 1; else hi = mid;
            }
            // rows without chunks share their first-chunk number with the next row: step back to the
            // row that owns c (the last one at or before c that has chunks is the one found: a row
            // without chunks has the same number as its successor, so the search ends behind them)
            const int32_t row = lo - 1;
            const int32_t first = s_mc[row], next = row + 1 < (int32_t)n_rows ? s_mc[row + 1] : total;
            p.rec[c] = make_int4(row, c - first, next - first, s_len[row]);
        }
    }
    if (threadIdx.x < 2 * kDealers) p.deal[threadIdx.x * kDealerStride] = 0;
    if (threadIdx.x == 0) {
        int32_t items = carry[0];
        for (int q = 0; q < kSingleClasses; ++q) { p.counts[4 + q] = carry[1 + q]; items += carry[1 + q]; }
        p.mc_off[n_rows] = carry[0];
        p.counts[0] = items;
        p.counts[1] = carry[0];
        p.counts[2] = 0;
        p.counts[3] = fail_s;                         // rows left to the whole-row kernel (the seam kernel may add some)
    }
}

// The entries of the chunks of the chunked rows: one thread per row, a row of many chunks by its wave.
// The work list of a batch whose rows are about equally long and all taken whole: nothing but the
// counters; the rows are dealt in their given order (sorting them by length gains nothing then, and
// the scan over 16,384 rows by one workgroup takes 19 us).
__global__ void bpe_plan_in_order_kernel(int32_t n_rows, BpePlan p)
{
    if (threadIdx.x == 0) {
        p.counts[0] = n_rows;
        p.counts[1] = 0;
        p.counts[2] = 0;
        p.counts[3] = 0;
        for (int q = 0; q < kSingleClasses; ++q) p.counts[4 + q] = 0;
    }
    if (threadIdx.x < 2 * kDealers) p.deal[threadIdx.x * kDealerStride] = 0;
}

__global__ __launch_bounds__(256) void bpe_expand_kernel(const int64_t *__restrict__ offsets, int64_t n_rows,
                                                         BpePlan p)
{
    const int64_t row = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int lane = threadIdx.x & 63;
    int32_t mo = 0, nc = 0, len = 0;
    if (row < n_rows) {
        mo = p.mc_off[row];
        nc = p.mc_off[row + 1] - mo;                 // 0 for a row that is a single item
        len = (int32_t)(offsets[row + 1] - offsets[row]);
    }
    const bool big = nc > 8;
    if (!big)
        for (int32_t k = 0; k < nc; ++k) p.rec[mo + k] = make_int4((int32_t)row, k, nc, len);
    uint64_t todo = __ballot(big);
    while (todo) {
        const int src = __builtin_amdgcn_readfirstlane(__builtin_ctzll(todo));
        todo &= todo - 1;
        const int32_t b_row = __builtin_amdgcn_readlane((int32_t)row, src);
        const int32_t b_mo = __builtin_amdgcn_readlane(mo, src), b_nc = __builtin_amdgcn_readlane(nc, src);
        const int32_t b_len = __builtin_amdgcn_readlane(len, src);
        for (int32_t k = lane; k < b_nc; k += 64) p.rec[b_mo + k] = make_int4(b_row, k, b_nc, b_len);
    }
}

// Rows and chunks of at most CAP bytes, state in LDS (15 bytes per position); the merge table
// stays in global memory (L2-resident) and is probed in batches.  NT = 64: every wave of the
// workgroup takes its own item (no workgroup barrier after the set-up); NT = blockDim.x: the
// workgroup shares an item.  PLANNED: the items are those of the work list (rows and chunks of
// long rows), handed out through an atomic counter.  Otherwise (no row of the batch is longer
// than CAP) an item is a row, teams take rows round robin, and no work list is built at all.
// CHUNKS = false: the list holds whole rows only (no row of the batch is cut), and the kernel is
// built without the chunk path, whose copy of the engine costs it registers (a workgroup per CU
// for rows of at most 1 KB).
// PADDED: a row's ids go straight to its row of a.pad_ids, padded (dnatok_bpe_encode_padded).
// LDS of a workgroup of the engine kernel: the small tables, the work item, the reduction cells
// and 15 bytes of state per position and team.
template <int NT, int TEAMS, int CAP>
constexpr size_t lds_bytes()
{
    return kLeadBytes + 64 + (size_t)TEAMS * (4 * (NT / 64) + 4) * 4 + (size_t)TEAMS * CAP * 15 +
           (size_t)TEAMS * NT + 64;
}
// workgroups of a form that a CU's LDS holds
template <int NT, int TEAMS, int CAP>
constexpr int lds_workgroups_per_cu()
{
    return kLdsPieces / (int)((lds_bytes<NT, TEAMS, CAP>() + kLdsPiece - 1) / kLdsPiece);
}
static_assert(lds_workgroups_per_cu<256, 1, 2048>() == 5 && lds_workgroups_per_cu<64, 4, 512>() == 5 &&
              lds_workgroups_per_cu<256, 1, 1408>() == 7 && lds_workgroups_per_cu<256, 1, 1536>() == 6,
              "a form grew over a piece boundary of the LDS");

// Waves per SIMD that the compiler has to leave room for: as many as the LDS lets a CU hold (a
// workgroup is a wave on every SIMD).  Teams of four waves over rows of at most 1 KB are limited by
// registers, not by LDS (17 KB a team): 64 registers are eight teams per CU, 65 are seven, 73 six,
// and left to itself the compiler takes 72 to 85, depending on the form.  The forms that also cut
// rows into chunks hold a second copy of the engine and are left alone below 2 KB (test geometries);
// the forms with a wave per row stop at seven (the eighth wave costs them spills to memory).
#ifdef DNATOK_BPE_PHASE_CYCLES
template <int NT, int TEAMS, int CAP, bool CHUNKS>
constexpr int kBpeWaves = 1;              // (the phase clock's cells take registers: no limit in that build)
#else
template <int NT, int TEAMS, int CAP, bool CHUNKS>
constexpr int kBpeWaves = (CHUNKS && CAP < 2048) ? 1
                          : lds_workgroups_per_cu<NT, TEAMS, CAP>() < (NT == 256 ? 8 : 7)
                                ? lds_workgroups_per_cu<NT, TEAMS, CAP>() : (NT == 256 ? 8 : 7);
#endif

template <int NT, int TEAMS, int CAP, bool PLANNED, bool LTAB = false, bool CHARS = false, bool CHUNKS = PLANNED,
          bool PADDED = false>
__global__ __launch_bounds__(NT *TEAMS) __attribute__((amdgpu_waves_per_eu(kBpeWaves<NT, TEAMS, CAP, CHUNKS>)))
void bpe_lds_kernel(
    BpeArgs a /* stays the first parameter: kernel_args_now() reads it from the start of the argument segment */,
    const uint8_t *__restrict__ bytes, const int64_t *__restrict__ offsets,
    BpePlan p, int32_t n_rows, int32_t *__restrict__ tok_tmp, int32_t *__restrict__ lengths)
{
    extern __shared__ __align__(16) uint8_t smem[];
    uint8_t *sp = smem;
    const PairTable pt{a.tab, a.shift, a.mul1, a.mul2};
    // the rules between single bytes by byte class, when the table has few enough such bytes, or
    // else the byte-to-symbol table, in the same place
    uint16_t *b2s = reinterpret_cast<uint16_t *>(sp);
    FirstPairs *const first_lds = reinterpret_cast<FirstPairs *>(sp); sp += kLeadBytes;
    static_assert(kLeadBytes % 16 == 0, "the state arrays behind it stay aligned");
    if (a.first) {
        const uint32_t *src = reinterpret_cast<const uint32_t *>(a.first);
        for (int i = threadIdx.x; i < (int)(sizeof(FirstPairs) / 4); i += NT * TEAMS)
            reinterpret_cast<uint32_t *>(first_lds)[i] = src[i];
    } else {
        for (int i = threadIdx.x; i < 256; i += NT * TEAMS) b2s[i] = a.byte_to_sym[i];
    }
    const FirstPairs *const first_pairs = a.first ? first_lds : nullptr;
    const int team = threadIdx.x / NT, tid = threadIdx.x % NT;
    int32_t *next_item = reinterpret_cast<int32_t *>(sp) + team; sp += 16 * sizeof(int32_t);
    uint32_t *red = reinterpret_cast<uint32_t *>(sp) + team * (4 * (NT / 64) + 4); sp += TEAMS * (4 * (NT / 64) + 4) * 4;
    PosRec<uint16_t> *P = reinterpret_cast<PosRec<uint16_t> *>(sp) + (size_t)team * CAP; sp += (size_t)TEAMS * CAP * 8;
    uint32_t *PG = reinterpret_cast<uint32_t *>(sp) + (size_t)team * CAP; sp += (size_t)TEAMS * CAP * 4;   // product | gate << 16
    uint16_t *Q = reinterpret_cast<uint16_t *>(sp) + (size_t)team * (CAP / 2); sp += (size_t)TEAMS * CAP;
    uint16_t *C = reinterpret_cast<uint16_t *>(sp) + (size_t)team * CAP; sp += (size_t)TEAMS * CAP * 2;
    uint8_t *D = sp + (size_t)team * NT; sp += (size_t)TEAMS * NT;
    // LTAB: the workgroup keeps the compact form of the merge table in LDS (a copy per workgroup,
    // brought in with 16-byte loads before the first row)
    uint32_t *ltab = nullptr;
    if (LTAB) {
        ltab = reinterpret_cast<uint32_t *>(smem + ((sp - smem + 15) & ~(ptrdiff_t)15));
        const uint4 *src4 = reinterpret_cast<const uint4 *>(a.ltab);
        uint4 *dst4 = reinterpret_cast<uint4 *>(ltab);
        for (int i = threadIdx.x; i < kLdsTabWords / 4; i += NT * TEAMS) dst4[i] = src4[i];
    }
    const LdsPairTable lpt{ltab, ltab + kLdsTabSlots, a.lmul1, a.lmul2};
    __syncthreads();

    const int32_t n_shortest = PLANNED ? p.counts[4 + kSingleClasses - 1] : 0;
    const int32_t n_items = !PLANNED ? n_rows
                            : (a.part == 2 ? n_shortest : p.counts[0] - (a.part == 1 ? n_shortest : 0));
    int32_t *const deal = PLANNED ? p.deal + (a.part == 2 ? kDealers * kDealerStride : 0) : nullptr;
    static_assert(PLANNED || !CHUNKS, "chunks come from the work list");
    static_assert(!(CHARS && NT == 256) || CAP >= 1024, "the merge queue holds the table of single-character ids (1 KB)");
    static_assert(!PADDED || (!CHUNKS && !LTAB), "padded rows: whole rows");
    const int32_t n_mc = CHUNKS ? p.counts[1] : 0;
    const int32_t n_single0 = PLANNED ? p.counts[4] : 0, n_single1 = PLANNED ? p.counts[5] : 0;
    // A team's first item is its own number; only the items beyond one per team are handed out
    // through the counter.  (Every team asking the counter at the start of the kernel is a
    // thousand atomics on one address, about 12 ns each, before the last team has its row.)
    const int32_t n_teams = (int32_t)gridDim.x * TEAMS;
    int32_t item = (int32_t)blockIdx.x * TEAMS + team;
    int32_t left = 0;                                // items of the team's current share still to come
    const int32_t dealer = item & (a.dealers - 1);
    // the first item beyond the teams' own that this team's counter hands out
    const int32_t dealt_from = n_teams + ((dealer - n_teams) & (a.dealers - 1));
    constexpr bool padded = PADDED;
    int32_t team_longest = 0;                        // (padded) most tokens in a row of this team
    for (bool first = true;; first = false) {
        if (!first) {
            if (PLANNED && left > 0) {               // (the same in every lane)
                item += a.dealers;
                --left;
            } else if (PLANNED) {
                if (n_teams >= n_items) break;       // nothing was left for the counters
                if (tid == 0)
                    *next_item = dealt_from + a.dealers * atomicAdd(&deal[dealer * kDealerStride], a.grab);
                team_sync<NT>();
                item = *next_item;
                team_sync<NT>();
                left = a.grab - 1;
            } else {
                item += n_teams;
            }
        }
        if (item >= n_items) break;
        int32_t row = item, k = 0, nc = 1;
        if (PLANNED) {
            if (CHUNKS && item < n_mc) {
                const int4 rc = p.rec[item];
                row = rc.x; k = rc.y; nc = rc.z;
            } else if (!CHUNKS && a.in_order) {
                row = item;
            } else if (!CHUNKS && a.part == 2) {
                row = p.single[kSingleClasses - 1][item];
            } else {
                int32_t j = item - n_mc;
                const int32_t *list = p.single[0];
                if (j >= n_single0) {
                    j -= n_single0; list = p.single[1];
                    if (j >= n_single1) { j -= n_single1; list = p.single[2]; }
                }
                row = list[j];
            }
        }
        // (a team is whole waves: its item is the same in every lane, and so is all that follows from it)
        row = __builtin_amdgcn_readfirstlane(row);
        k = __builtin_amdgcn_readfirstlane(k);
        nc = __builtin_amdgcn_readfirstlane(nc);
        const int64_t start = offsets[row];
        const int64_t len = offsets[row + 1] - start;
        // one straight path per iteration (no `continue`): every lane of the team must come
        // back to the fetch above together, or lanes that skipped ahead would re-read the
        // old item while lane 0 has not fetched the next one yet
        if ((!CHUNKS || nc == 1) && (len > CAP || len <= 0)) {
            // too long: left to the whole-row kernel (row_fail is set); empty: no tokens
            if (tid == 0) lengths[row] = len > CAP ? -1 : 0;
            if (padded) {
                const BpeArgsInMemory ka = kernel_args_now();
                const int64_t stride = ka->pad_stride;
                const int32_t elem = ka->pad_elem, pad_id = ka->pad_id;
                void *const ids = ka->pad_ids;
                uint8_t *const mask = ka->pad_mask;
                for (int64_t i = tid; i < stride; i += NT) {
                    const int64_t at = (int64_t)row * stride + i;
                    if (elem == 4) reinterpret_cast<int32_t *>(ids)[at] = pad_id;
                    else if (elem == 8) reinterpret_cast<int64_t *>(ids)[at] = (int64_t)pad_id;
                    else if (elem == 2) reinterpret_cast<int16_t *>(ids)[at] = (int16_t)pad_id;
                    else reinterpret_cast<uint8_t *>(ids)[at] = (uint8_t)pad_id;
                    if (mask) mask[at] = 0;
                }
            }
            if (CHARS) {
                for (int64_t i = tid; i < len; i += NT) {
                    a.char_ids[start + i] = a.char_lut[bytes[start + i]];
                    if (a.char_mask) a.char_mask[start + i] = 1;
                }
            }
        } else if (!CHUNKS || nc == 1) {
            if (LTAB)
                bpe_row<NT, uint16_t, (CAP + NT - 1) / NT>(lpt, b2s, a.out_remap, bytes + start, (int)len, P, PG,
                                      Q, C, D, red, tid, tok_tmp + start, lengths + row, nullptr, 0, 0, nullptr,
                                      nullptr, nullptr, nullptr, 0, 0, first_pairs, 0, a.byte_to_sym);
            else {
                const int32_t n_tok = bpe_row<NT, uint16_t, (CAP + NT - 1) / NT, CHARS, PADDED>(
                    pt, b2s, a.out_remap, bytes + start, (int)len, P, PG, Q, C, D, red, tid,
                    padded ? nullptr : tok_tmp + start,        // (a padded row finds its own cells)
                    lengths + row, nullptr, 0, 0, nullptr, a.char_lut, CHARS ? a.char_ids + start : nullptr,
                    CHARS && a.char_mask ? a.char_mask + start : nullptr, 0, (int)len, first_pairs, row,
                    a.byte_to_sym);
                team_longest = n_tok > team_longest ? n_tok : team_longest;
            }
        } else if (CHUNKS) {
            const int64_t e0 = (int64_t)k * p.core - p.overlap < 0 ? 0 : (int64_t)k * p.core - p.overlap;
            int64_t e1 = (int64_t)(k + 1) * p.core + p.overlap;
            if (e1 > len) e1 = len;
            const int32_t m = item;                  // chunk items come first in the list
            uint16_t *raw = p.chunk_sym + (size_t)m * p.ext;
            // what the chunk shares with no other: from the end of the left overlap to the start of the right one
            int64_t mid_lo = k > 0 ? (int64_t)k * p.core + p.overlap : 0;
            if (mid_lo > len) mid_lo = len;
            const int64_t mid_hi = k + 1 < nc ? (int64_t)(k + 1) * p.core - p.overlap : len;
            // the single-character ids of a long row are written chunk by chunk: every chunk those of its core
            const int64_t core_hi = (int64_t)(k + 1) * p.core < len ? (int64_t)(k + 1) * p.core : len;
            bpe_row<NT, uint16_t, (CAP + NT - 1) / NT, CHARS>(
                pt, b2s, a.out_remap, bytes + start + e0, (int)(e1 - e0), P, PG, Q, C, D, red, tid, nullptr,
                nullptr, raw, (int)(mid_lo - e0), (int)(mid_hi - e0), p.cnt + 4 * (size_t)m, a.char_lut,
                CHARS ? a.char_ids + start + e0 : nullptr, CHARS && a.char_mask ? a.char_mask + start + e0 : nullptr,
                (int)((int64_t)k * p.core - e0), (int)(core_hi - e0), first_pairs, 0, a.byte_to_sym);
        }
        team_sync<NT>();
    }
    // (padded) every workgroup reports once, whether it had a row or not
    const BpeArgsInMemory ka = kernel_args_now();
    if (padded && ka->max_tree) {
        if (TEAMS == 1) {
            if (threadIdx.x == 0) publish_max(ka->max_tree, (unsigned)team_longest, ka->longest);
        } else {
            __shared__ int32_t s_longest[TEAMS];
            if (tid == 0) s_longest[team] = team_longest;
            __syncthreads();                         // (every team has left its loop)
            if (threadIdx.x == 0) {
                int32_t m = 0;
#pragma unroll
                for (int q = 0; q < TEAMS; ++q) m = s_longest[q] > m ? s_longest[q] : m;
                publish_max(ka->max_tree, (unsigned)m, ka->longest);
            }
        }
    }
}

// The seam between a chunk of a multi-chunk row and the chunk to its right, by a team of NT threads
// (256 / NT teams to a workgroup).  The two runs over the shared stretch (2 x overlap positions) are
// staged in the team's part of LDS first: the search walks from token start to token start, a chain
// of dependent reads that is several times shorter there than in L2.  A seam is two dependent trips
// to memory and a few hundred instructions.  With few seams (all of them resident at once as
// workgroups: one batch of 32 rows of 100 kbp) the 256-thread team is faster (the call 160 against
// 165 us: the per-lane loops are a quarter as long).  With many, what counts is the number of seams in
// flight, and a wave per seam holds four times as many, with no workgroup barrier (8 such batches per
// call: 56 -> 38 us, 8 ragged batches of 12 Mbp: 97 -> 56 us).
constexpr int kSeamStage = 1024;          // positions of the shared stretch a team holds in LDS
constexpr int kSeamWaveFrom = 2048;       // from this many chunk slots on: a wave per seam

template <int NT>
__global__ __launch_bounds__(256) void bpe_seam_kernel(const int64_t *__restrict__ offsets, BpePlan p)
{
    constexpr int TEAMS = 256 / NT;
    __shared__ uint16_t stage_s[TEAMS][2 * kSeamStage];
    __shared__ uint32_t red_s[TEAMS][4 * (NT / 64) + 4];
    const int team = threadIdx.x / NT, tid = threadIdx.x % NT;
    const int wv = (NT == 64) ? 0 : (tid >> 6);
    uint16_t *const sa_s = stage_s[team], *const sb_s = stage_s[team] + kSeamStage;
    uint32_t *const red = red_s[team];
    // (the first record is requested beside the count, not behind it; the slot exists either way)
    const int32_t m0 = (int32_t)blockIdx.x * TEAMS + team;
    int4 rc_first = make_int4(0, 0, 0, 0);
    if ((int64_t)m0 < p.max_mc) rc_first = p.rec[m0];
    const int32_t n_mc = p.counts[1];
    for (int32_t m = m0; m < n_mc; m += (int32_t)gridDim.x * TEAMS) {
        const int4 rc = m == m0 ? rc_first : p.rec[m];
        const int32_t row = rc.x, k = rc.y, nc = rc.z;
        if (k + 1 >= nc) continue;                                   // last chunk: no seam to the right (the same for the whole team)
        const int64_t len = rc.w;
        const int64_t ea0 = (int64_t)k * p.core - p.overlap < 0 ? 0 : (int64_t)k * p.core - p.overlap;
        int64_t ea1 = (int64_t)(k + 1) * p.core + p.overlap;
        if (ea1 > len) ea1 = len;
        const int64_t eb0 = (int64_t)(k + 1) * p.core - p.overlap;
        const uint16_t *A = p.chunk_sym + (size_t)m * p.ext;         // A[i - ea0]
        const uint16_t *B = p.chunk_sym + (size_t)(m + 1) * p.ext;   // B[i - eb0]
        const int n = (int)(ea1 - eb0);                              // shared positions eb0 .. ea1
        const bool staged = n <= kSeamStage;                         // (the same for the whole team)
        team_sync<NT>();                                             // the team's last seam is read no more
        if (staged) {
            for (int j = tid; j < n; j += NT) { sa_s[j] = A[eb0 - ea0 + j]; sb_s[j] = B[j]; }
            team_sync<NT>();
        }
        // (two instances, one reading LDS and one reading memory: a choice per read would be a
        // flat load from a selected address)
        auto search = [&](auto a_at, auto b_at) {
        uint32_t mine = 0xFFFFFFFFu;
        for (int i = tid; i < n; i += NT) {
            const uint32_t sa = a_at(i);
            if (sa == kNone || sa != b_at(i)) continue;
            int j = i + 1;                                           // next token start in A
            while (j < n && a_at(j) == kNone) ++j;
            if (j < n && a_at(j) == b_at(j)) { mine = (uint32_t)(eb0 + j); break; }
        }
        uint32_t b, unused;
        team_min2<NT>(mine, kEmptyKey, red, wv, b, unused);
        if (tid == 0) {
            if (b == 0xFFFFFFFFu) {
                p.seam[m] = -1;
                if (atomicExch(&p.row_fail[row], 1) == 0) atomicAdd(&p.counts[3], 1);
            } else {
                p.seam[m] = (int32_t)b;
            }
        }
        // tokens of A in the shared stretch left of the seam, tokens of B right of it: with each
        // chunk's own count of its unshared stretch these are the chunks' shares of the row
        uint32_t tail = 0, head = 0;
        if (b != 0xFFFFFFFFu) {
            const int cut = (int)((int64_t)b - eb0);
            for (int i = tid; i < n; i += NT) {
                if (i < cut) tail += a_at(i) != kNone;
                else head += b_at(i) != kNone;
            }
        }
        team_sync<NT>();                                 // (red is still being read for the minimum)
        uint32_t both;                                   // (each count is below 2^16: one sum for the two)
        (void)team_exclusive_sum<NT>(tail | (head << 16), red, wv, both);
        if (tid == 0) {
            p.cnt[4 * (size_t)m + 2] = (int32_t)(both & 0xFFFFu);
            p.cnt[4 * (size_t)(m + 1) + 1] = (int32_t)(both >> 16);
        }
        };
        if (staged)
            search([&](int j) -> uint32_t { return sa_s[j]; }, [&](int j) -> uint32_t { return sb_s[j]; });
        else
            search([&](int j) -> uint32_t { return A[eb0 - ea0 + j]; }, [&](int j) -> uint32_t { return B[j]; });
    }
}

// The same search for shared stretches of at most kSeamMaskSpan positions (twice the shipped
// overlap), a wave per seam, with no walk from token start to token start and no staging: position
// 64 q + lane of the stretch is lane's in pass q, a ballot per pass gives the token starts of A, those
// of B, and the starts of A whose token is the same in B, as 64-bit masks that every lane holds.
// A seam is a start j of A that matches and whose previous start of A matches too: the previous
// start is the highest set bit below j in the mask of its pass, or the last start of the passes
// before (a running value that is the same in all lanes).  The counts the gather needs are popcounts
// of the masks on either side of the seam.  A seam is then one trip to memory behind its record and
// some hundred instructions; the walks were chains of dependent LDS reads, a token long each.
constexpr int kSeamMaskSpan = 256;

__global__ __launch_bounds__(256) void bpe_seam_mask_kernel(BpePlan p)
{
    constexpr int kPasses = kSeamMaskSpan / 64;
    const int team = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int32_t n_mc = p.counts[1];
    for (int64_t m64 = (int64_t)blockIdx.x * 4 + team; m64 < n_mc; m64 += (int64_t)gridDim.x * 4) {
        const int32_t m = (int32_t)m64;
        const int4 rc = p.rec[m];
        const int32_t row = rc.x, k = rc.y, nc = rc.z;
        if (k + 1 >= nc) continue;                                   // last chunk: no seam to the right (the same for the whole wave)
        const int64_t len = rc.w;
        const int64_t ea0 = (int64_t)k * p.core - p.overlap < 0 ? 0 : (int64_t)k * p.core - p.overlap;
        int64_t ea1 = (int64_t)(k + 1) * p.core + p.overlap;
        if (ea1 > len) ea1 = len;
        const int64_t eb0 = (int64_t)(k + 1) * p.core - p.overlap;
        const uint16_t *A = p.chunk_sym + (size_t)m * p.ext + (eb0 - ea0);       // A[i], B[i]: position eb0 + i
        const uint16_t *B = p.chunk_sym + (size_t)(m + 1) * p.ext;
        const int n = (int)(ea1 - eb0);                              // shared positions, at most kSeamMaskSpan
        uint32_t sa[kPasses], sb[kPasses];
#pragma unroll
        for (int q = 0; q < kPasses; ++q) {
            const int i = 64 * q + lane;
            sa[q] = i < n ? (uint32_t)A[i] : kNone;
            sb[q] = i < n ? (uint32_t)B[i] : kNone;
        }
        uint64_t starts_a[kPasses], starts_b[kPasses];
        int seam = -1;                                               // position within the stretch
        bool last_start_matches = false;                             // the last start of A in the passes so far: is it one of B's, same token?
#pragma unroll
        for (int q = 0; q < kPasses; ++q) {
            const uint64_t s_a = __ballot(sa[q] != kNone);
            const uint64_t same = __ballot(sa[q] != kNone && sa[q] == sb[q]);
            starts_a[q] = s_a;
            starts_b[q] = __ballot(sb[q] != kNone);
            // the previous start of A before this lane's position
            const uint64_t below = s_a & ((1ull << lane) - 1ull);
            const bool prev_matches = below ? (same >> (63 - __builtin_clzll(below)) & 1ull) != 0 : last_start_matches;
            const uint64_t ok = __ballot(sa[q] != kNone && sa[q] == sb[q] && prev_matches);
            if (seam < 0 && ok) seam = 64 * q + __builtin_ctzll(ok);
            if (s_a) last_start_matches = (same >> (63 - __builtin_clzll(s_a)) & 1ull) != 0;
        }
        // (a matched first start of the stretch with no start before it is no seam: the walk began at
        // a matched start and took the next one)
        uint32_t tail = 0, head = 0;                                 // tokens of A left of the seam, of B from the seam on
        if (seam >= 0) {
#pragma unroll
            for (int q = 0; q < kPasses; ++q) {
                const int lo = seam - 64 * q;                        // bits below lo belong to A's side
                const uint64_t left = lo <= 0 ? 0ull : (lo >= 64 ? ~0ull : ((1ull << lo) - 1ull));
                tail += (uint32_t)__builtin_popcountll(starts_a[q] & left);
                head += (uint32_t)__builtin_popcountll(starts_b[q] & ~left);
            }
        }
        if (lane == 0) {
            if (seam < 0) {
                p.seam[m] = -1;
                if (atomicExch(&p.row_fail[row], 1) == 0) atomicAdd(&p.counts[3], 1);
            } else {
                p.seam[m] = (int32_t)(eb0 + seam);
            }
            p.cnt[4 * (size_t)m + 2] = (int32_t)tail;
            p.cnt[4 * (size_t)(m + 1) + 1] = (int32_t)head;
        }
    }
}

// The part of a row that chunk k contributes: from the seam on its left to the seam on its right.
struct ChunkSpan {
    int32_t row, k, nc;
    int64_t lo, hi, e0;       // owned row positions [lo, hi); e0 = row position of the chunk's first symbol
};

__device__ __forceinline__ ChunkSpan chunk_span(const BpePlan &p, int32_t m)
{
    ChunkSpan c;
    const int4 rc = p.rec[m];
    c.row = rc.x; c.k = rc.y; c.nc = rc.z;
    const int64_t len = rc.w;
    c.e0 = (int64_t)c.k * p.core - p.overlap < 0 ? 0 : (int64_t)c.k * p.core - p.overlap;
    c.lo = c.k > 0 ? p.seam[m - 1] : 0;
    c.hi = c.k + 1 < c.nc ? p.seam[m] : len;
    return c;
}

// A team of NT threads per chunk (256 / NT teams to a workgroup): its tokens, compacted, behind those
// of the row's earlier chunks.  Positions are taken NT at a time: a ballot per wave places every live
// symbol among its wave's, the waves' counts go through LDS, all symbols (and their remapped ids) of a
// block of passes are loaded before the first store, and a wave's stores go to consecutive cells.  (A
// contiguous piece per thread with load, remap and store in one loop ran as a chain of dependent
// loads: the stores may alias what the next iteration reads.)  As with the seams: a 256-thread team
// when all chunks are resident at once anyway, a wave per chunk (four times as many in flight) when
// there are many.
template <int NT>
__global__ __launch_bounds__(256) void bpe_gather_kernel(
    BpeArgs a, const int64_t *__restrict__ offsets, BpePlan p, int32_t *__restrict__ tok_tmp,
    int32_t *__restrict__ lengths)
{
    constexpr int kPasses = 8;
    constexpr int TEAMS = 256 / NT, NW = NT / 64;
    __shared__ uint32_t red_s[TEAMS][4 * NW + 4];
    __shared__ uint32_t wave_cnt_s[TEAMS][kPasses][NW];
    const int team = threadIdx.x / NT, tid = threadIdx.x % NT;
    const int wv = (NT == 64) ? 0 : (tid >> 6), lane = tid & 63;
    uint32_t *const red = red_s[team];
    uint32_t (*const wave_cnt)[NW] = wave_cnt_s[team];
    const int32_t n_mc = p.counts[1];
    for (int32_t m = (int32_t)blockIdx.x * TEAMS + team; m < n_mc; m += (int32_t)gridDim.x * TEAMS) {
        const ChunkSpan c = chunk_span(p, m);
        if (p.row_fail[c.row]) continue;                 // (the same for the whole team)
        // tokens of the row's chunks before this one.  (Summing them behind the first block's
        // loads instead of in front of them made the kernel 10 % slower; requesting the chunk's
        // record beside the chunk count, and both seams beside the record, 5 %.)
        uint32_t before = 0;
        for (int32_t j = tid; j < c.k; j += NT) {
            const int32_t *part = p.cnt + 4 * (size_t)(m - c.k + j);       // {unshared, after left seam, before right seam}
            before += (uint32_t)(part[0] + (j > 0 ? part[1] : 0) + part[2]);
        }
        uint32_t base;
        (void)team_exclusive_sum<NT>(before, red, wv, base);
        const uint16_t *sym = p.chunk_sym + (size_t)m * p.ext;
        int32_t *out = tok_tmp + offsets[c.row];
        uint32_t done = base;
        for (int64_t i0 = c.lo; i0 < c.hi; i0 += kPasses * NT) {
            uint32_t sy[kPasses], ahead[kPasses];
            int32_t val[kPasses];
#pragma unroll
            for (int k = 0; k < kPasses; ++k) {
                const int64_t i = i0 + k * NT + tid;
                sy[k] = i < c.hi ? (uint32_t)sym[i - c.e0] : kNone;
            }
#pragma unroll
            for (int k = 0; k < kPasses; ++k) {
                val[k] = (sy[k] != kNone && a.out_remap) ? a.out_remap[sy[k]] : (int32_t)sy[k];
                const uint64_t live = __ballot(sy[k] != kNone);
                ahead[k] = lanes_below(live);
                if (lane == 0) wave_cnt[k][wv] = (uint32_t)__builtin_popcountll(live);
            }
            team_sync<NT>();
            uint32_t at = done;
#pragma unroll
            for (int k = 0; k < kPasses; ++k) {
                uint32_t mine = at;
#pragma unroll
                for (int w = 0; w < NW; ++w) {
                    const uint32_t n = wave_cnt[k][w];
                    if (w < wv) mine += n;
                    at += n;
                }
                if (sy[k] != kNone) out[mine + ahead[k]] = val[k];
            }
            done = at;
            team_sync<NT>();                                 // wave_cnt is rewritten by the next block
        }
        if (tid == 0 && c.k + 1 == c.nc) lengths[c.row] = (int32_t)done;
    }
}

// The same with a wave per chunk that holds the whole chunk at once (chunks of at most kGatherExt
// symbols, a multiple of eight): lane L takes the 32 symbols from 32 L on, four 16-byte loads whose
// addresses depend on the chunk's number alone, so they are under way before the chunk's record
// has arrived; seams, the row's place and the counts of the earlier chunks are then one more trip
// together.  The lanes' live symbols (those inside the chunk's span) are compacted through the
// wave's part of LDS, and the ids go out 64 consecutive cells at a time.  A chunk is two to three
// trips to memory; with a block of eight passes per trip it was a dozen (8 ragged batches of 12 Mbp:
// 93 -> 82 us, 8 batches of 32 x 100 kbp: 24 -> 20 us).
constexpr int kGatherExt = 2048;

__global__ __launch_bounds__(256) void bpe_gather_wave_kernel(
    BpeArgs a, const int64_t *__restrict__ offsets, BpePlan p, int32_t *__restrict__ tok_tmp,
    int32_t *__restrict__ lengths)
{
    __shared__ uint16_t compact_s[4][kGatherExt];
    const int team = threadIdx.x >> 6, lane = threadIdx.x & 63;
    uint16_t *const compact = compact_s[team];
    const int32_t n_mc = p.counts[1];
    for (int64_t m64 = (int64_t)blockIdx.x * 4 + team; m64 < p.max_mc; m64 += (int64_t)gridDim.x * 4) {
        const int32_t m = (int32_t)m64;
        // the lane's 32 symbols (beyond the chunk's end: none)
        const uint4 *src = reinterpret_cast<const uint4 *>(p.chunk_sym + (size_t)m * p.ext);
        uint4 g[4];
#pragma unroll
        for (int q = 0; q < 4; ++q)
            g[q] = lane * 32 + q * 8 < p.ext ? src[lane * 4 + q] : uint4{~0u, ~0u, ~0u, ~0u};
        const int4 rc = p.rec[m];
        if (m >= n_mc) break;                            // (the same for the whole wave)
        const int32_t row = rc.x, k = rc.y, nc = rc.z;
        const int64_t len = rc.w;
        const int64_t e0 = (int64_t)k * p.core - p.overlap < 0 ? 0 : (int64_t)k * p.core - p.overlap;
        // second trip: the seams, the row's state and place, the earlier chunks' counts
        const int32_t seam_l = k > 0 ? p.seam[m - 1] : 0;
        const int32_t seam_r = k + 1 < nc ? p.seam[m] : 0;
        const int32_t failed = p.row_fail[row];
        const int64_t row_at = offsets[row];
        uint32_t before = 0;
        for (int32_t j = lane; j < k; j += 64) {
            const int4 part = *reinterpret_cast<const int4 *>(p.cnt + 4 * (size_t)(m - k + j));   // {unshared, after left seam, before right seam, -}
            before += (uint32_t)(part.x + (j > 0 ? part.y : 0) + part.z);
        }
        if (failed) continue;                            // (the same for the whole wave)
        const uint32_t inc_b = wave_inclusive_sum_u32(before);
        const uint32_t base = (uint32_t)__builtin_amdgcn_readlane((int)inc_b, 63);
        const int64_t lo = k > 0 ? (int64_t)seam_l : 0, hi = k + 1 < nc ? (int64_t)seam_r : len;
        // which of the lane's positions lie in [lo, hi) and start a token
        const int64_t p0 = e0 + lane * 32;
        uint32_t in_span = ~0u;
        if (lo > p0) in_span = lo - p0 >= 32 ? 0u : (~0u << (uint32_t)(lo - p0));
        if (hi < p0 + 32) in_span &= hi <= p0 ? 0u : (~0u >> (uint32_t)(p0 + 32 - hi));
        const uint32_t w[16] = {g[0].x, g[0].y, g[0].z, g[0].w, g[1].x, g[1].y, g[1].z, g[1].w,
                                g[2].x, g[2].y, g[2].z, g[2].w, g[3].x, g[3].y, g[3].z, g[3].w};
        uint32_t live = 0;
#pragma unroll
        for (int q = 0; q < 16; ++q) {
            live |= ((w[q] & 0xFFFFu) != kNone ? 1u : 0u) << (2 * q);
            live |= ((w[q] >> 16) != kNone ? 1u : 0u) << (2 * q + 1);
        }
        live &= in_span;
        const uint32_t mine = (uint32_t)__builtin_popcount(live);
        const uint32_t inc = wave_inclusive_sum_u32(mine);
        const uint32_t total = (uint32_t)__builtin_amdgcn_readlane((int)inc, 63);
        uint32_t at = inc - mine;
#pragma unroll
        for (int q = 0; q < 32; ++q) {
            if (live >> q & 1u) compact[at++] = (uint16_t)(q & 1 ? w[q >> 1] >> 16 : w[q >> 1] & 0xFFFFu);
        }
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
        int32_t *const out = tok_tmp + row_at + base;
#pragma unroll 4
        for (uint32_t t = lane; t < total; t += 64) {
            const uint32_t sy = compact[t];
            out[t] = a.out_remap ? a.out_remap[sy] : (int32_t)sy;
        }
        if (lane == 0 && k + 1 == nc) lengths[row] = (int32_t)(base + total);
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();                 // the wave's part of LDS is rewritten by its next chunk
    }
}

// Whole-row kernel for rows above the LDS capacity that could not be chunked: one workgroup per
// row, state in global scratch (26 bytes / base).
template <int NT>
__global__ __launch_bounds__(NT) void bpe_long_kernel(
    BpeArgs a, const uint8_t *__restrict__ bytes, const int64_t *__restrict__ offsets,
    int64_t n_rows, int64_t max_len, BpePlan p, int32_t *__restrict__ tok_tmp,
    int32_t *__restrict__ lengths)
{
    __shared__ uint32_t red[4 * (NT / 64) + 4];
    __shared__ uint8_t D[NT];
    __shared__ uint16_t b2s[256];
    if (p.counts[3] == 0) return;                    // no row needs this kernel (the usual case)
    for (int i = threadIdx.x; i < 256; i += NT) b2s[i] = a.byte_to_sym[i];
    __syncthreads();
    // each workgroup owns one slab of scratch, sized for the longest row
    uint8_t *slab = p.slabs + (size_t)blockIdx.x * p.slab_bytes;
    const PairTable pt{a.tab, a.shift, a.mul1, a.mul2};
    for (int64_t row = blockIdx.x; row < n_rows; row += gridDim.x) {
        if (!p.row_fail[row]) continue;
        const int64_t start = offsets[row];
        const int64_t len = offsets[row + 1] - start;
        if (len > max_len) {                     // longer than the caller declared: no room in the slab
            if (threadIdx.x == 0) lengths[row] = -1;
            continue;
        }
        const size_t n = ((size_t)len + 7) & ~(size_t)7;
        PosRec<uint32_t> *P = reinterpret_cast<PosRec<uint32_t> *>(slab);
        uint32_t *PG = reinterpret_cast<uint32_t *>(P + n);      // product | gate << 16
        uint32_t *Q = PG + n;                                    // n / 2 entries
        uint32_t *C = Q + n / 2;                                 // n entries
        bpe_row<NT, uint32_t, 0>(pt, b2s, a.out_remap, bytes + start, (int)len, P, PG,
                              Q, C, D, red, threadIdx.x, tok_tmp + start, lengths + row);
        __syncthreads();
    }
}

}  // namespace dnatok

using namespace dnatok;

extern "C" int dnatok_bpe_table_create(const int32_t *byte_to_id_h, const int32_t *pair_a_h,
                                       const int32_t *pair_b_h, const int32_t *new_id_h,
                                       int32_t n_merges, int32_t n_symbols,
                                       const int32_t *out_remap_h, dnatok_bpe_t **out)
{
    DNATOK_REQUIRE(byte_to_id_h && out && (n_merges == 0 || (pair_a_h && pair_b_h && new_id_h)),
                   DNATOK_E_INVALID, "dnatok_bpe_table_create: null argument");
    DNATOK_REQUIRE(n_merges >= 0 && n_symbols > 0, DNATOK_E_INVALID,
                   "dnatok_bpe_table_create: bad sizes");
    DNATOK_REQUIRE(n_symbols <= 65535 && n_merges <= 65534, DNATOK_E_TOO_LARGE,
                   "dnatok_bpe_table_create: %d symbols / %d merges exceed the 16-bit state",
                   n_symbols, n_merges);
    for (int i = 0; i < 256; ++i)
        DNATOK_REQUIRE(byte_to_id_h[i] >= 0 && byte_to_id_h[i] < n_symbols, DNATOK_E_INVALID,
                       "dnatok_bpe_table_create: byte_to_id[%d] out of range", i);
    for (int32_t i = 0; i < n_merges; ++i) {
        const int32_t pa = pair_a_h[i], pb = pair_b_h[i], nid = new_id_h[i];
        DNATOK_REQUIRE(pa >= 0 && pa < n_symbols && pb >= 0 && pb < n_symbols && nid >= 0 && nid < n_symbols,
                       DNATOK_E_INVALID, "dnatok_bpe_table_create: merge %d has an id out of range", i);
    }
    // Four to eight slots per rule, far below the load at which two-choice cuckoo placement starts
    // to fail; a placement that still fails is redone with other multipliers, then a larger table.
    static const uint32_t kMul[8] = {0x9E3779B1u, 0x85EBCA6Bu, 0xC2B2AE35u, 0x27D4EB2Fu,
                                     0x165667B1u, 0xD3A2646Du, 0xFD7046C5u, 0xB55A4F09u};
    uint32_t slots = 64, shift = 26, mul1 = 0, mul2 = 0;
    while (slots < (uint32_t)n_merges * 4u + 2u) { slots <<= 1; --shift; }
    std::vector<uint4> tab;
    std::vector<uint32_t> first_use;                           // lowest rank using a symbol
    // A pair listed more than once counts with its last entry: HF collects the merges into a map
    // in list order, so a later entry replaces the rank and product of an earlier one.
    std::unordered_map<uint32_t, int32_t> last_entry;
    last_entry.reserve((size_t)n_merges * 2);
    for (int32_t i = 0; i < n_merges; ++i)
        last_entry[((uint32_t)pair_a_h[i] << 16) | (uint32_t)pair_b_h[i]] = i;
    for (int attempt = 0;; ++attempt) {
        DNATOK_REQUIRE(shift > 4, DNATOK_E_INVALID, "dnatok_bpe_table_create: the merge table could not be hashed");
        mul1 = kMul[(2 * attempt) & 7]; mul2 = kMul[(2 * attempt + 1) & 7];
        tab.assign(slots, uint4{kEmptyKey, kNone, 0, 0});
        first_use.assign(n_symbols, 0xFFFFFFFFu);
        bool placed = true;
        for (int32_t i = 0; i < n_merges && placed; ++i) {
            const uint32_t pa = (uint32_t)pair_a_h[i], pb = (uint32_t)pair_b_h[i];
            const uint32_t key = (pa << 16) | pb;
            if (last_entry[key] != i) continue;        // replaced by a later entry of the same pair
            if (first_use[pa] == 0xFFFFFFFFu) first_use[pa] = (uint32_t)i;
            if (first_use[pb] == 0xFFFFFFFFu) first_use[pb] = (uint32_t)i;
            uint4 e{key, (uint32_t)i, (uint32_t)new_id_h[i], 0};
            uint32_t came_from = 0xFFFFFFFFu;
            placed = false;
            for (int kick = 0; kick < 512; ++kick) {
                const uint32_t h1 = pair_slot(e.x, mul1, shift), h2 = pair_slot(e.x, mul2, shift);
                if (tab[h1].x == kEmptyKey) { tab[h1] = e; placed = true; break; }
                if (tab[h2].x == kEmptyKey) { tab[h2] = e; placed = true; break; }
                const uint32_t v = (h1 == came_from) ? h2 : h1;     // push out the entry of the other slot
                const uint4 out_e = tab[v];
                tab[v] = e; e = out_e; came_from = v;
            }
        }
        if (placed) break;
        if ((attempt & 3) == 3) { slots <<= 1; --shift; }
    }
    int monotone = 1;
    for (int32_t i = 0; i < n_merges; ++i) {
        const uint32_t key = ((uint32_t)pair_a_h[i] << 16) | (uint32_t)pair_b_h[i];
        if (last_entry[key] == i && first_use[new_id_h[i]] <= (uint32_t)i) monotone = 0;
    }
    for (uint4 &e : tab)
        if (e.x != kEmptyKey) {
            const uint32_t fu = first_use[e.z];
            e.z |= (fu == 0xFFFFFFFFu ? kNone : fu) << 16;
        }
    std::vector<uint16_t> b2s(256);
    for (int i = 0; i < 256; ++i) b2s[i] = (uint16_t)byte_to_id_h[i];

    // the compact form for LDS (see LdsPairTable), when symbols and ranks fit 12 bits
    std::vector<uint32_t> ltab;
    uint32_t lmul1 = 0, lmul2 = 0;
    if (n_symbols <= 8192 && n_merges <= kLdsTabRanks - 1 && n_merges > 0) {
        static const uint32_t kMul24[6] = {0x29E3779u, 0x185EBCBu, 0x3C2B2AFu, 0x227D4EBu, 0x1165667u, 0x2D3A265u};   // odd, 26 bits
        for (int attempt = 0; attempt < 3 && ltab.empty(); ++attempt) {
            lmul1 = kMul24[2 * attempt]; lmul2 = kMul24[2 * attempt + 1];
            std::vector<uint32_t> slot(kLdsTabSlots, 0), key_of(kLdsTabSlots, 0), pg(kLdsTabRanks, kNone | (kNone << 16));
            bool placed = true;
            for (int32_t i = 0; i < n_merges && placed; ++i) {
                const uint32_t pa = (uint32_t)pair_a_h[i], pb = (uint32_t)pair_b_h[i];
                if (last_entry[(pa << 16) | pb] != i) continue;
                const uint32_t fu = first_use[new_id_h[i]];
                pg[i] = (uint32_t)new_id_h[i] | ((fu == 0xFFFFFFFFu ? kNone : fu) << 16);
                uint32_t key = (pa << 13) | pb, rank = (uint32_t)i, came_from = 0xFFFFFFFFu;
                placed = false;
                for (int kick = 0; kick < 512; ++kick) {
                    const uint32_t h1 = lds_pair_hash(key, lmul1), h2 = lds_pair_hash(key, lmul2);
                    const uint32_t s1 = h1 >> 13, s2 = h2 >> 13;
                    const uint32_t w1 = (rank << 15) | ((h1 & 0x1FFFu) << 2) | 1u, w2 = (rank << 15) | ((h2 & 0x1FFFu) << 2) | 3u;
                    if (slot[s1] == 0) { slot[s1] = w1; key_of[s1] = key; placed = true; break; }
                    if (slot[s2] == 0) { slot[s2] = w2; key_of[s2] = key; placed = true; break; }
                    const uint32_t v = (s1 == came_from) ? s2 : s1;        // push out the rule of the other slot
                    const uint32_t out_key = key_of[v], out_rank = slot[v] >> 15;
                    slot[v] = v == s1 ? w1 : w2; key_of[v] = key;
                    key = out_key; rank = out_rank; came_from = v;
                }
            }
            if (placed) {
                ltab = slot;
                ltab.insert(ltab.end(), pg.begin(), pg.end());
            }
        }
    }

    // FirstPairs: the rules whose two symbols both stand for single bytes, by classes of bytes
    FirstPairs first{};
    bool have_first = false;
    {
        std::vector<int> cls_of_sym(n_symbols, -1);
        std::vector<uint8_t> byte_sym(n_symbols, 0);
        for (int v = 0; v < 256; ++v) byte_sym[b2s[v]] = 1;
        std::vector<uint32_t> members;                        // symbols with a class, in class order
        auto give_class = [&](uint32_t sym) {
            if (cls_of_sym[sym] < 0) { cls_of_sym[sym] = (int)members.size(); members.push_back(sym); }
        };
        for (int32_t i = 0; i < n_merges; ++i) {
            const uint32_t pa = (uint32_t)pair_a_h[i], pb = (uint32_t)pair_b_h[i];
            if (last_entry[(pa << 16) | pb] != i || !byte_sym[pa] || !byte_sym[pb]) continue;
            give_class(pa);
            give_class(pb);
        }
        if ((int)members.size() <= kFirstClasses) {
            have_first = true;
            for (int v = 0; v < 256; ++v) {
                const uint32_t c = cls_of_sym[b2s[v]] < 0 ? kNoClass : (uint32_t)cls_of_sym[b2s[v]];
                first.cls4[v >> 1] |= (uint8_t)(c << ((v & 1) * 4));
            }
            for (size_t c = 0; c < members.size(); ++c) first.sym[c] = (uint16_t)members[c];
            for (int q = 0; q < kFirstClasses * kFirstClasses; ++q) first.rule[q] = uint2{kNone, kNone | (kNone << 16)};
            for (size_t ca = 0; ca < members.size(); ++ca)
                for (size_t cb = 0; cb < members.size(); ++cb) {
                    const uint32_t key = (members[ca] << 16) | members[cb];
                    const uint4 &e1 = tab[pair_slot(key, mul1, shift)], &e2 = tab[pair_slot(key, mul2, shift)];
                    const uint4 *hit = e1.x == key ? &e1 : (e2.x == key ? &e2 : nullptr);
                    if (hit) first.rule[ca * kFirstClasses + cb] = uint2{hit->y, hit->z};
                }
        }
    }

    auto up = [](size_t v) { return (v + 255) & ~(size_t)255; };
    const size_t o_tab = 0;
    const size_t o_b2s = up(o_tab + (size_t)slots * sizeof(uint4));
    const size_t o_remap = up(o_b2s + 512);
    const size_t o_first = up(o_remap + (out_remap_h ? (size_t)n_symbols * 4 : 0));
    const size_t o_ltab = up(o_first + sizeof(FirstPairs));
    const size_t o_trees = up(o_ltab + ltab.size() * 4);
    const size_t total = up(o_trees + (size_t)kMaxTreeSlots * kTreeWords * 8) + 256;
    std::vector<uint8_t> host(total, 0);             // (the trees start as zeros)
    memcpy(&host[o_tab], tab.data(), (size_t)slots * sizeof(uint4));
    memcpy(&host[o_b2s], b2s.data(), 512);
    if (out_remap_h) memcpy(&host[o_remap], out_remap_h, (size_t)n_symbols * 4);
    if (!ltab.empty()) memcpy(&host[o_ltab], ltab.data(), ltab.size() * 4);
    memcpy(&host[o_first], &first, sizeof(FirstPairs));
    void *blob = nullptr;
    hipError_t e = hipMalloc(&blob, total);
    if (e == hipSuccess) e = hipMemcpy(blob, host.data(), total, hipMemcpyHostToDevice);
    if (e != hipSuccess) {
        set_error("dnatok_bpe_table_create: %s", hipGetErrorString(e));
        if (blob) (void)hipFree(blob);
        return DNATOK_E_HIP;
    }
    dnatok_bpe_table *t = new dnatok_bpe_table();
    uint8_t *b = (uint8_t *)blob;
    t->n_merges = n_merges; t->n_symbols = n_symbols; t->slots = slots; t->shift = shift; t->mul1 = mul1; t->mul2 = mul2;
    t->monotone = monotone; t->blob = blob;
    t->tab = (uint4 *)(b + o_tab);
    t->byte_to_sym = (uint16_t *)(b + o_b2s);
    t->out_remap = out_remap_h ? (int32_t *)(b + o_remap) : nullptr;
    t->ltab = ltab.empty() ? nullptr : (uint32_t *)(b + o_ltab);
    t->lmul1 = lmul1; t->lmul2 = lmul2;
    t->first = have_first ? (void *)(b + o_first) : nullptr;
    t->max_trees = (unsigned long long *)(b + o_trees);
    *out = t;
    return DNATOK_OK;
}

extern "C" int dnatok_bpe_table_set_chunk_geometry(dnatok_bpe_t *t, int32_t core, int32_t overlap)
{
    DNATOK_REQUIRE(t, DNATOK_E_INVALID, "dnatok_bpe_table_set_chunk_geometry: null table");
    DNATOK_REQUIRE((core == 0 && overlap == 0) ||
                       (core >= 256 && overlap >= 32 && core > 2 * overlap && core + 2 * overlap <= kLdsCap),
                   DNATOK_E_INVALID,
                   "dnatok_bpe_table_set_chunk_geometry: need core >= 256, overlap >= 32, core > 2 * overlap, "
                   "core + 2 * overlap <= %d (or 0, 0 for the shipped geometry)", kLdsCap);
    t->chunk_core.store(core, std::memory_order_relaxed);
    t->chunk_overlap.store(overlap, std::memory_order_relaxed);
    return DNATOK_OK;
}

extern "C" int dnatok_bpe_table_set_placement(dnatok_bpe_t *t, int32_t mode)
{
    DNATOK_REQUIRE(t, DNATOK_E_INVALID, "dnatok_bpe_table_set_placement: null table");
    DNATOK_REQUIRE(mode >= 0 && mode <= 2, DNATOK_E_INVALID, "dnatok_bpe_table_set_placement: mode is 0, 1 or 2");
    t->placement.store(mode, std::memory_order_relaxed);
    return DNATOK_OK;
}

extern "C" void dnatok_bpe_table_destroy(dnatok_bpe_t *t)
{
    if (!t) return;
    if (t->blob) (void)hipFree(t->blob);
    delete t;
}

extern "C" size_t dnatok_bpe_scratch_bytes(const dnatok_bpe_t *t, int64_t n_rows, int64_t max_len,
                                           int64_t total)
{
    if (n_rows <= 0) return 256;
    return make_plan(t, nullptr, n_rows, max_len, total).total_bytes;
}

namespace {

// Longest row (negative lengths count as 0) by one workgroup: where no tree of atomics carries it.
__global__ __launch_bounds__(1024) void bpe_longest_kernel(const int32_t *__restrict__ lengths, int64_t n_rows,
                                                           int32_t *__restrict__ longest)
{
    __shared__ uint32_t red[16];
    uint32_t m = 0;
    for (int64_t i = threadIdx.x; i < n_rows; i += 1024) {
        const int32_t v = lengths[i];
        m = v > 0 && (uint32_t)v > m ? (uint32_t)v : m;
    }
    m = wave_max_u32(m);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = m;
    __syncthreads();
    if (threadIdx.x == 0) {
        uint32_t all = 0;
        for (int w = 0; w < 16; ++w) all = all > red[w] ? all : red[w];
        *longest = (int32_t)all;
    }
}


// Teams of the LDS kernel that are resident at once: of the form that works through a list with
// chunks, which holds the most registers (a batch of more rows than that gets a list).
template <int NT, int TEAMS, int CAP>
int64_t lds_resident_teams()
{
    static const int resident =
        resident_workgroups(bpe_lds_kernel<NT, TEAMS, CAP, true>, NT * TEAMS, lds_bytes<NT, TEAMS, CAP>(), 2);
    return (int64_t)resident * TEAMS;
}

template <int NT, int TEAMS, int CAP, bool PLANNED, bool CHARS = false, bool CHUNKS = PLANNED, bool PADDED = false>
int launch_lds_as(const BpeArgs &a, const uint8_t *bytes, const int64_t *offsets, const BpePlan &p,
                  int64_t n_rows, int32_t *tok_tmp, int32_t *lengths, hipStream_t s)
{
    const size_t lds = lds_bytes<NT, TEAMS, CAP>();
    auto kern = bpe_lds_kernel<NT, TEAMS, CAP, PLANNED, false, CHARS, CHUNKS, PADDED>;
    // (once per kernel form; two threads that both find it unset both set it, to the same value)
    static std::atomic<bool> attr_set{false};
    if (!attr_set.load(std::memory_order_acquire)) {
        DNATOK_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        attr_set.store(true, std::memory_order_release);
    }
    const int64_t items = PLANNED ? p.max_items : n_rows;
    int64_t grid = (items + TEAMS - 1) / TEAMS;
    static const int64_t resident = resident_workgroups(kern, NT * TEAMS, lds, 2);    // (of this form)
    if (grid > resident) grid = resident;
    if (a.max_tree && grid > kTreeRows) grid = kTreeRows;
    if (grid < 1) grid = 1;
    // a team's share per trip to its work counter: one item, and with very many items 1/32 of
    // what a team takes in all, at most 8 (the last shares decide how evenly the teams end)
    BpeArgs a2 = a;
    const int64_t per_team = PLANNED ? (items - grid * TEAMS) / (grid * TEAMS * 32) : 1;
    a2.grab = (int32_t)(per_team < 1 ? 1 : (per_team > 8 ? 8 : per_team));
    // several counters for the wave-sized teams of short rows (thousands of teams, items of a few
    // microseconds); one for the 256-thread teams, whose items last far longer than a turn at the
    // counter and end most evenly when any team may take the last of them
    a2.dealers = TEAMS > 1 ? kDealers : 1;
    while (a2.dealers > grid * TEAMS) a2.dealers >>= 1;
    kern<<<(int)grid, NT * TEAMS, lds, s>>>(a2, bytes, offsets, p, (int32_t)n_rows, tok_tmp, lengths);
    DNATOK_HIP_TRY(hipGetLastError());
    return DNATOK_OK;
}

// Where the merge table is kept (dnatok_bpe_set_table_placement): 0 = in global memory (L2), always;
// 1 = the compact form in LDS when the table has one, no row is longer than 1024 bytes and the batch
// leaves the room for it (at most one row per team resident with the table's 48 KB added to every
// workgroup); 2 = the compact form for every such batch, whatever its size.  0 is the default because
// it measured faster: bringing 48 KB into every workgroup costs more than the lookups save (256 rows
// of 1 KB: 23.8 us against 25.1 us with the table in LDS, 512 rows: 25.7 against 26.7; 1024 rows, which
// then need two rounds of workgroups: 30.4 against 49.4).
// The unplanned 1 KB form of the LDS kernel with the compact table in LDS.
template <int NT, int TEAMS, int CAP>
int64_t ltab_resident_teams()
{
    static const int resident = resident_workgroups(bpe_lds_kernel<NT, TEAMS, CAP, false, true>, NT * TEAMS,
                                                    lds_bytes<NT, TEAMS, CAP>() + kLdsTabWords * 4 + 16, 1);
    return (int64_t)resident * TEAMS;
}

template <int NT, int TEAMS, int CAP>
int launch_lds_ltab(const BpeArgs &a, const uint8_t *bytes, const int64_t *offsets, const BpePlan &p,
                    int64_t n_rows, int32_t *tok_tmp, int32_t *lengths, hipStream_t s)
{
    const size_t lds = lds_bytes<NT, TEAMS, CAP>() + kLdsTabWords * 4 + 16;
    auto kern = bpe_lds_kernel<NT, TEAMS, CAP, false, true>;
    // (once per kernel form; two threads that both find it unset both set it, to the same value)
    static std::atomic<bool> attr_set{false};
    if (!attr_set.load(std::memory_order_acquire)) {
        DNATOK_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        attr_set.store(true, std::memory_order_release);
    }
    int64_t grid = (n_rows + TEAMS - 1) / TEAMS;
    const int64_t resident = ltab_resident_teams<NT, TEAMS, CAP>() / TEAMS;
    if (grid > resident) grid = resident;
    if (grid < 1) grid = 1;
    kern<<<(int)grid, NT * TEAMS, lds, s>>>(a, bytes, offsets, p, (int32_t)n_rows, tok_tmp, lengths);
    DNATOK_HIP_TRY(hipGetLastError());
    return DNATOK_OK;
}

// The work list (plan) is needed when rows are cut into chunks or left to the whole-row kernel,
// and when there are more rows than resident teams: rows then are dealt through the list's
// counter, since rows take different times and a fixed share per team ends in a long tail
// (16 x 1024 rows of 1 KB: 0.60 ms with fixed shares, 0.46 ms dealt).  A batch of at most one row
// per team needs neither list nor counter.
template <int NT, int TEAMS, int CAP>
int run_lds_part(bool long_rows, int chunking, bool force_plan, const BpeArgs &a, const uint8_t *bytes,
                 const int64_t *offsets, const BpePlan &p, int64_t n_rows, int32_t *tok_tmp, int32_t *lengths,
                 hipStream_t s)
{
    if constexpr (CAP == 1024) {
        // (only for a batch that one launch encodes whole: with force_plan or a part of a split
        // batch the work list decides which rows a launch takes, and this form has none)
        if (!long_rows && !force_plan && a.part == 0 && a.ltab && !a.char_ids && !a.pad_ids) {
            const int mode = a.placement;
            if (mode == 2 || (mode == 1 && n_rows <= ltab_resident_teams<NT, TEAMS, 1024>()))
                return launch_lds_ltab<NT, TEAMS, 1024>(a, bytes, offsets, p, n_rows, tok_tmp, lengths, s);
        }
    }
    const bool planned = long_rows || force_plan || n_rows > lds_resident_teams<NT, TEAMS, CAP>();
    if (planned) {
        if (a.in_order) {                            // (no row is cut)
            bpe_plan_in_order_kernel<<<1, 64, 0, s>>>((int32_t)n_rows, p);
            DNATOK_HIP_TRY(hipGetLastError());
        } else {
            const int expand_here = chunking >> 1;
            if (n_rows >= kPlanTiledFrom) {
                const int tiles = (int)((n_rows + kPlanTile - 1) / kPlanTile);
                bpe_plan_kernel<1><<<tiles, 1024, 0, s>>>(offsets, n_rows, chunking & 1, 0, p);
                DNATOK_HIP_TRY(hipGetLastError());
                bpe_plan_kernel<2><<<tiles, 1024, 0, s>>>(offsets, n_rows, chunking & 1, 0, p);
            } else {
                bpe_plan_kernel<0><<<1, 1024, 0, s>>>(offsets, n_rows, chunking & 1, expand_here, p);
            }
            DNATOK_HIP_TRY(hipGetLastError());
            if ((chunking & 1) && !expand_here) {
                bpe_expand_kernel<<<(int)((n_rows + 255) / 256), 256, 0, s>>>(offsets, n_rows, p);
                DNATOK_HIP_TRY(hipGetLastError());
            }
        }
        if (chunking & 1) {
            if (a.char_ids) return launch_lds_as<NT, TEAMS, CAP, true, true>(a, bytes, offsets, p, n_rows, tok_tmp, lengths, s);
            return launch_lds_as<NT, TEAMS, CAP, true>(a, bytes, offsets, p, n_rows, tok_tmp, lengths, s);
        }
        if (a.pad_ids) return launch_lds_as<NT, TEAMS, CAP, true, false, false, true>(a, bytes, offsets, p, n_rows, tok_tmp, lengths, s);
        if (a.char_ids) return launch_lds_as<NT, TEAMS, CAP, true, true, false>(a, bytes, offsets, p, n_rows, tok_tmp, lengths, s);
        return launch_lds_as<NT, TEAMS, CAP, true, false, false>(a, bytes, offsets, p, n_rows, tok_tmp, lengths, s);
    }
    if (a.pad_ids) return launch_lds_as<NT, TEAMS, CAP, false, false, false, true>(a, bytes, offsets, p, n_rows, tok_tmp, lengths, s);
    if (a.char_ids) return launch_lds_as<NT, TEAMS, CAP, false, true>(a, bytes, offsets, p, n_rows, tok_tmp, lengths, s);
    return launch_lds_as<NT, TEAMS, CAP, false>(a, bytes, offsets, p, n_rows, tok_tmp, lengths, s);
}

template <int NT, int TEAMS, int CAP>
int run_lds(bool long_rows, int chunking, bool split, const BpeArgs &a_in, const uint8_t *bytes, const int64_t *offsets,
            const BpePlan &p, int64_t n_rows, int32_t *tok_tmp, int32_t *lengths, hipStream_t s)
{
    // split: the rows of the shortest class (at most a quarter of an extended chunk: 512 bytes) get
    // a launch of their own with teams of one wave, after the launch for everything else
    BpeArgs a = a_in;
    a.part = split ? 1 : 0;
    if (split) {
        BpeArgs b = a_in;
        b.part = 2;
        const int rc = run_lds_part<NT, TEAMS, CAP>(long_rows, chunking, true, a, bytes, offsets, p, n_rows, tok_tmp, lengths, s);
        if (rc) return rc;
        if (b.pad_ids) return launch_lds_as<64, 4, 512, true, false, false, true>(b, bytes, offsets, p, n_rows, tok_tmp, lengths, s);
        if (b.char_ids) return launch_lds_as<64, 4, 512, true, true, false>(b, bytes, offsets, p, n_rows, tok_tmp, lengths, s);
        return launch_lds_as<64, 4, 512, true, false, false>(b, bytes, offsets, p, n_rows, tok_tmp, lengths, s);
    }
    return run_lds_part<NT, TEAMS, CAP>(long_rows, chunking, false, a, bytes, offsets, p, n_rows, tok_tmp, lengths, s);
}

}  // namespace

// The launches of one encode call; p lies inside a scratch buffer that holds p.total_bytes.
static int bpe_encode_launch(const dnatok_bpe_t *t, const uint8_t *bytes, const int64_t *offsets, int64_t n_rows,
                             int64_t max_len, int64_t total, const BpePlan &p, int32_t *tok_tmp, int32_t *lengths, hipStream_t s,
                             const int32_t *char_lut = nullptr, int32_t *char_ids = nullptr,
                             uint8_t *char_mask = nullptr, const BpeArgs *padded = nullptr)
{
    BpeArgs a{t->tab, t->byte_to_sym, t->out_remap, t->shift, t->mul1, t->mul2, t->n_merges, t->ltab, t->lmul1, t->lmul2,
              t->first, char_lut, char_ids, char_mask};
    a.placement = t->placement.load(std::memory_order_relaxed);
    if (padded) {
        a.pad_ids = padded->pad_ids; a.pad_mask = padded->pad_mask; a.pad_remap = padded->pad_remap;
        a.pad_elem = padded->pad_elem; a.pad_left = padded->pad_left;
        a.pad_stride = padded->pad_stride; a.pad_id = padded->pad_id;
        a.max_tree = padded->max_tree; a.longest = padded->longest;
    }

    const bool long_rows = max_len > p.ext;
    // rows of about one length (the mean at least 3/4 of the longest), none cut: dealt in their given
    // order; and so are very many short rows of any lengths (sorting 100,000 of them costs the one
    // workgroup that does it 115 us, their unsorted end at most the time of one row, about 25 us)
    a.in_order = !long_rows && (total >= (max_len * n_rows / 4) * 3 || (max_len <= 512 && n_rows >= 8192)) ? 1 : 0;
    int chunking = (long_rows && t->monotone) ? 1 : 0;
    // bit 1: the plan kernel writes the chunk entries itself (few rows, few chunks: one launch less)
    if (chunking && n_rows <= kPlanInlineRows && p.max_mc <= kPlanInlineChunks) chunking |= 2;
    // the LDS capacity variant follows the longest row (or the chunk size for longer rows):
    // less LDS per workgroup means more workgroups per CU
    int rc;
    const int64_t work_len = max_len < p.ext ? max_len : p.ext;    // longest piece the LDS kernel sees
    // Mostly short rows with some long ones among them (the mean at most 384 bytes, the longest above
    // 512): the short ones, which a 256-thread team would take as long over as over a row of 1 KB,
    // get a launch of their own.  The two launches cannot both carry the longest row up the one
    // tree: it is taken from the lengths afterwards.
    const bool split = work_len > 512 && n_rows >= 1024 && total / n_rows <= 384 && p.ext / 4 <= 512;
    int32_t *const longest_after = split && a.max_tree ? a.longest : nullptr;
    if (split) {
        a.in_order = 0;
        a.max_tree = nullptr;
    }
    // short rows: a wave per row, four rows to a workgroup (a 256-thread team would leave most of
    // its lanes without a position, and a row's time is its rounds, not its length)
    if (work_len <= 256)         rc = run_lds<64, 4, 256>(long_rows, chunking, split, a, bytes, offsets, p, n_rows, tok_tmp, lengths, s);
    else if (work_len <= 384)    rc = run_lds<64, 4, 384>(long_rows, chunking, split, a, bytes, offsets, p, n_rows, tok_tmp, lengths, s);
    else if (work_len <= 512)    rc = run_lds<64, 4, 512>(long_rows, chunking, split, a, bytes, offsets, p, n_rows, tok_tmp, lengths, s);
    else if (work_len <= 1024)   rc = run_lds<256, 1, 1024>(long_rows, chunking, split, a, bytes, offsets, p, n_rows, tok_tmp, lengths, s);
    else if (work_len <= 1408)   rc = run_lds<256, 1, 1408>(long_rows, chunking, split, a, bytes, offsets, p, n_rows, tok_tmp, lengths, s);
    else if (work_len <= 1536)   rc = run_lds<256, 1, 1536>(long_rows, chunking, split, a, bytes, offsets, p, n_rows, tok_tmp, lengths, s);
    else if (work_len <= 2048)   rc = run_lds<256, 1, 2048>(long_rows, chunking, split, a, bytes, offsets, p, n_rows, tok_tmp, lengths, s);
    else                         rc = run_lds<256, 1, kLdsCap>(long_rows, chunking, split, a, bytes, offsets, p, n_rows, tok_tmp, lengths, s);
    if (rc) return rc;
    if (long_rows) {
        if (chunking) {
            int64_t g = p.max_mc < 4096 ? p.max_mc : 4096;
            if (2 * p.overlap <= kSeamMaskSpan) {                          // a wave per seam, the search on ballots
                int64_t gs = (p.max_mc + 3) / 4;
                bpe_seam_mask_kernel<<<(int)(gs > 4096 ? 4096 : gs), 256, 0, s>>>(p);
            } else if (p.max_mc >= kSeamWaveFrom) {                        // a wave per seam, up to two rounds of workgroups
                int64_t gs = (p.max_mc + 3) / 4;
                bpe_seam_kernel<64><<<(int)(gs > 4096 ? 4096 : gs), 256, 0, s>>>(offsets, p);
            } else {
                bpe_seam_kernel<256><<<(int)(g < 1 ? 1 : g), 256, 0, s>>>(offsets, p);
            }
            DNATOK_HIP_TRY(hipGetLastError());
            if (p.max_mc >= kSeamWaveFrom) {
                int64_t gs = (p.max_mc + 3) / 4;
                if (p.ext <= kGatherExt && p.ext % 8 == 0)
                    bpe_gather_wave_kernel<<<(int)(gs > 4096 ? 4096 : gs), 256, 0, s>>>(a, offsets, p, tok_tmp, lengths);
                else
                    bpe_gather_kernel<64><<<(int)(gs > 4096 ? 4096 : gs), 256, 0, s>>>(a, offsets, p, tok_tmp, lengths);
            } else {
                bpe_gather_kernel<256><<<(int)(g < 1 ? 1 : g), 256, 0, s>>>(a, offsets, p, tok_tmp, lengths);
            }
            DNATOK_HIP_TRY(hipGetLastError());
        }
        bpe_long_kernel<kLongThreads><<<p.n_slabs, kLongThreads, 0, s>>>(a, bytes, offsets, n_rows, max_len, p,
                                                                        tok_tmp, lengths);
        DNATOK_HIP_TRY(hipGetLastError());
    }
    if (longest_after) {
        bpe_longest_kernel<<<1, 1024, 0, s>>>(lengths, n_rows, longest_after);
        DNATOK_HIP_TRY(hipGetLastError());
    }
    return DNATOK_OK;
}

static int bpe_encode_check(const char *who, const dnatok_bpe_t *t, const uint8_t *bytes, const int64_t *offsets,
                            int64_t n_rows, int64_t max_len, int64_t total, const int32_t *tok_tmp,
                            const int32_t *lengths)
{
    DNATOK_REQUIRE(t && offsets && lengths, DNATOK_E_INVALID, "%s: null argument", who);
    DNATOK_REQUIRE(n_rows >= 0 && max_len >= 0 && total >= 0, DNATOK_E_INVALID, "%s: negative size", who);
    DNATOK_REQUIRE(max_len < (int64_t)1 << 31 && total / 256 + n_rows < (int64_t)1 << 30, DNATOK_E_TOO_LARGE,
                   "%s: batch too large for 32-bit work indices", who);
    DNATOK_REQUIRE(n_rows == 0 || total == 0 || (bytes && tok_tmp), DNATOK_E_INVALID, "%s: null buffer", who);
    return DNATOK_OK;
}

extern "C" int dnatok_bpe_encode(const dnatok_bpe_t *t, const uint8_t *bytes, const int64_t *offsets,
                                 int64_t n_rows, int64_t max_len, int64_t total, void *scratch,
                                 size_t scratch_bytes, int32_t *tok_tmp, int32_t *lengths, void *stream)
{
    const int bad = bpe_encode_check("dnatok_bpe_encode", t, bytes, offsets, n_rows, max_len, total, tok_tmp, lengths);
    if (bad) return bad;
    if (n_rows == 0) return DNATOK_OK;
    const BpePlan need = make_plan(t, nullptr, n_rows, max_len, total);
    DNATOK_REQUIRE(scratch && scratch_bytes >= need.total_bytes, DNATOK_E_SCRATCH,
                   "dnatok_bpe_encode: scratch holds %zu bytes, %zu needed", scratch_bytes, need.total_bytes);
    DNATOK_REQUIRE(((uintptr_t)scratch & 255) == 0, DNATOK_E_INVALID, "dnatok_bpe_encode: scratch must be 256-byte aligned");
    const BpePlan p = make_plan(t, (uint8_t *)scratch, n_rows, max_len, total);
    return bpe_encode_launch(t, bytes, offsets, n_rows, max_len, total, p, tok_tmp, lengths, (hipStream_t)stream);
}

extern "C" int dnatok_bpe_encode_with_chars(const dnatok_bpe_t *t, const uint8_t *bytes, const int64_t *offsets,
                                            int64_t n_rows, int64_t max_len, int64_t total, void *scratch,
                                            size_t scratch_bytes, int32_t *tok_tmp, int32_t *lengths,
                                            const int32_t *char_lut, int32_t *char_ids, uint8_t *char_mask,
                                            void *stream)
{
    const int bad = bpe_encode_check("dnatok_bpe_encode_with_chars", t, bytes, offsets, n_rows, max_len, total, tok_tmp,
                                     lengths);
    if (bad) return bad;
    DNATOK_REQUIRE(char_lut && (char_ids || total == 0), DNATOK_E_INVALID,
                   "dnatok_bpe_encode_with_chars: char_lut and char_ids are required");
    if (n_rows == 0) return DNATOK_OK;
    const BpePlan need = make_plan(t, nullptr, n_rows, max_len, total);
    DNATOK_REQUIRE(scratch && scratch_bytes >= need.total_bytes, DNATOK_E_SCRATCH,
                   "dnatok_bpe_encode_with_chars: scratch holds %zu bytes, %zu needed", scratch_bytes, need.total_bytes);
    DNATOK_REQUIRE(((uintptr_t)scratch & 255) == 0, DNATOK_E_INVALID,
                   "dnatok_bpe_encode_with_chars: scratch must be 256-byte aligned");
    const BpePlan p = make_plan(t, (uint8_t *)scratch, n_rows, max_len, total);
    return bpe_encode_launch(t, bytes, offsets, n_rows, max_len, total, p, tok_tmp, lengths, (hipStream_t)stream, char_lut,
                             char_ids, char_mask);
}

extern "C" int64_t dnatok_bpe_padded_direct_max(const dnatok_bpe_t *t)
{
    int core, overlap;
    chunk_geometry(t, &core, &overlap, 0, 0);
    return (int64_t)core + 2 * overlap;
}

extern "C" int dnatok_bpe_encode_padded_as(const dnatok_bpe_t *t, const uint8_t *bytes, const int64_t *offsets,
                                           int64_t n_rows, int64_t max_len, int64_t total, void *scratch,
                                           size_t scratch_bytes, int32_t *tok_tmp, const int32_t *remap, int32_t pad_id,
                                           int64_t stride, int pad_left, void *ids, int32_t id_bytes, uint8_t *mask,
                                           int32_t *lengths, int32_t *longest, void *stream)
{
    static const char *who = "dnatok_bpe_encode_padded_as";
    DNATOK_REQUIRE(id_bytes == 1 || id_bytes == 2 || id_bytes == 4 || id_bytes == 8, DNATOK_E_INVALID,
                   "%s: id_bytes must be 1, 2, 4 or 8", who);
    DNATOK_REQUIRE(t && offsets && (lengths || n_rows == 0), DNATOK_E_INVALID, "%s: null argument", who);
    DNATOK_REQUIRE(n_rows >= 0 && max_len >= 0 && total >= 0, DNATOK_E_INVALID, "%s: negative size", who);
    DNATOK_REQUIRE(max_len < (int64_t)1 << 31 && total / 256 + n_rows < (int64_t)1 << 30, DNATOK_E_TOO_LARGE,
                   "%s: batch too large", who);
    DNATOK_REQUIRE(stride >= 1 && stride < (int64_t)1 << 31, DNATOK_E_INVALID, "%s: stride must be in [1, 2^31)", who);
    DNATOK_REQUIRE(bytes || total == 0, DNATOK_E_INVALID, "%s: null bytes", who);
    DNATOK_REQUIRE(ids || n_rows == 0, DNATOK_E_INVALID, "%s: null ids", who);
    hipStream_t s = (hipStream_t)stream;
    if (n_rows == 0) {
        if (longest) {
            bpe_longest_kernel<<<1, 1024, 0, s>>>(lengths, 0, longest);
            DNATOK_HIP_TRY(hipGetLastError());
        }
        return DNATOK_OK;
    }
    const BpePlan need = make_plan(t, nullptr, n_rows, max_len, total);
    DNATOK_REQUIRE(scratch && scratch_bytes >= need.total_bytes, DNATOK_E_SCRATCH,
                   "%s: scratch holds %zu bytes, %zu needed", who, scratch_bytes, need.total_bytes);
    DNATOK_REQUIRE(((uintptr_t)scratch & 255) == 0, DNATOK_E_INVALID, "%s: scratch must be 256-byte aligned", who);
    const BpePlan p = make_plan(t, (uint8_t *)scratch, n_rows, max_len, total);
    if (max_len > p.ext) {
        // rows cut into chunks (or left to the whole-row kernel) are assembled in tok_tmp first
        DNATOK_REQUIRE(tok_tmp, DNATOK_E_INVALID,
                       "%s: a batch with a row of more than %d bytes needs tok_tmp (int32[total])", who, p.ext);
        const int rc = bpe_encode_launch(t, bytes, offsets, n_rows, max_len, total, p, tok_tmp, lengths, s);
        if (rc) return rc;
        if (longest) {
            bpe_longest_kernel<<<1, 1024, 0, s>>>(lengths, n_rows, longest);
            DNATOK_HIP_TRY(hipGetLastError());
        }
        return dnatok_pad_rows_as(tok_tmp, offsets, lengths, n_rows, remap, pad_id, stride, stride, 0, 0,
                                  pad_left ? 1 : 0, ids, id_bytes, mask, nullptr, nullptr, stream);
    }
    BpeArgs pad{};
    pad.pad_ids = ids; pad.pad_mask = mask; pad.pad_remap = remap; pad.pad_stride = stride; pad.pad_id = pad_id;
    pad.pad_elem = id_bytes; pad.pad_left = pad_left ? 1 : 0;
    pad.longest = longest;
    if (longest) {
        std::lock_guard<std::mutex> hold(t->slot_lock);
        auto it = t->slot_of_stream.find(stream);
        if (it == t->slot_of_stream.end() && (int)t->slot_of_stream.size() < kMaxTreeSlots)
            it = t->slot_of_stream.emplace(stream, (int)t->slot_of_stream.size()).first;
        if (it != t->slot_of_stream.end()) pad.max_tree = t->max_trees + (size_t)it->second * kTreeWords;
    }
    const int rc = bpe_encode_launch(t, bytes, offsets, n_rows, max_len, total, p, nullptr, lengths, s, nullptr, nullptr,
                                     nullptr, &pad);
    if (rc) return rc;
    if (longest && !pad.max_tree) {
        bpe_longest_kernel<<<1, 1024, 0, s>>>(lengths, n_rows, longest);
        DNATOK_HIP_TRY(hipGetLastError());
    }
    return DNATOK_OK;
}

extern "C" int dnatok_bpe_encode_padded(const dnatok_bpe_t *t, const uint8_t *bytes, const int64_t *offsets,
                                        int64_t n_rows, int64_t max_len, int64_t total, void *scratch,
                                        size_t scratch_bytes, int32_t *tok_tmp, const int32_t *remap, int32_t pad_id,
                                        int64_t stride, int32_t *ids, uint8_t *mask, int32_t *lengths,
                                        int32_t *longest, void *stream)
{
    return dnatok_bpe_encode_padded_as(t, bytes, offsets, n_rows, max_len, total, scratch, scratch_bytes, tok_tmp, remap,
                                       pad_id, stride, 0, ids, 4, mask, lengths, longest, stream);
}

// ---- the entry point that allocates nothing -------------------------------------------------
//
// The work buffer of dnatok_bpe_encode_static: one array in the code object's own device memory
// (each GPU the library runs on holds its copy until the process ends).  Host code never uses the
// array's name as an address: the address on the current device is asked for once per device.
constexpr size_t kStaticScratchBytes = DNATOK_BPE_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) uint8_t scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
static std::atomic<uint8_t *> g_static_scratch[kMaxDevices];

static int static_scratch_ptr(uint8_t **out)
{
    int dev = 0;
    DNATOK_HIP_TRY(hipGetDevice(&dev));
    DNATOK_REQUIRE(dev >= 0 && dev < kMaxDevices, DNATOK_E_INVALID,
                   "dnatok_bpe_encode_static: device index %d beyond %d", dev, kMaxDevices);
    uint8_t *ptr = g_static_scratch[dev].load(std::memory_order_acquire);
    if (!ptr) {
        // (two threads asking at once get the same answer; the address of a device's copy is fixed)
        void *sym = nullptr;
        DNATOK_HIP_TRY(hipGetSymbolAddress(&sym, HIP_SYMBOL(scratch)));
        DNATOK_REQUIRE(sym != nullptr, DNATOK_E_HIP, "dnatok_bpe_encode_static: no address for the work buffer");
        ptr = (uint8_t *)sym;
        g_static_scratch[dev].store(ptr, std::memory_order_release);
    }
    *out = ptr;
    return DNATOK_OK;
}

extern "C" size_t dnatok_bpe_static_scratch_bytes(void) { return kStaticScratchBytes; }

extern "C" int dnatok_bpe_encode_static(const dnatok_bpe_t *t, const uint8_t *bytes, const int64_t *offsets,
                                        int64_t n_rows, int64_t max_len, int64_t total,
                                        int32_t *tok_tmp, int32_t *lengths, void *stream)
{
    const int bad = bpe_encode_check("dnatok_bpe_encode_static", t, bytes, offsets, n_rows, max_len, total, tok_tmp,
                                     lengths);
    if (bad) return bad;
    if (n_rows == 0) return DNATOK_OK;
    // Fewer slabs for the whole-row fallback kernel (fewer rows redone at once) before giving up:
    // the slabs are what grows with the longest row.
    int64_t slabs = kLongGrid;
    BpePlan need = make_plan(t, nullptr, n_rows, max_len, total, slabs);
    while (need.total_bytes > kStaticScratchBytes && slabs > 1) {
        slabs /= 2;
        need = make_plan(t, nullptr, n_rows, max_len, total, slabs);
    }
    DNATOK_REQUIRE(need.total_bytes <= kStaticScratchBytes, DNATOK_E_TOO_LARGE,
                   "dnatok_bpe_encode_static: this batch needs %zu bytes of work space, the built-in buffer holds "
                   "%zu (use dnatok_bpe_encode with a caller-provided buffer)", need.total_bytes, kStaticScratchBytes);
    uint8_t *base = nullptr;
    const int rc = static_scratch_ptr(&base);
    if (rc) return rc;
    const BpePlan p = make_plan(t, base, n_rows, max_len, total, slabs);
    return bpe_encode_launch(t, bytes, offsets, n_rows, max_len, total, p, tok_tmp, lengths, (hipStream_t)stream);
}

#ifdef DNATOK_BPE_PHASE_CYCLES
// (measurement build only) The cells of all workgroups added up: cycles[0 .. 15], see BpePhase;
// reset != 0 clears them afterwards.  Synchronises the device.
extern "C" int dnatok_bpe_phase_cycles(unsigned long long *cycles, int reset)
{
    DNATOK_REQUIRE(cycles, DNATOK_E_INVALID, "dnatok_bpe_phase_cycles: null argument");
    std::vector<unsigned long long> all((size_t)kPhaseGroups * kPhaseCells);
    DNATOK_HIP_TRY(hipDeviceSynchronize());
    DNATOK_HIP_TRY(hipMemcpyFromSymbol(all.data(), HIP_SYMBOL(g_phase_cycles), all.size() * sizeof(unsigned long long)));
    for (int q = 0; q < kPhaseCells; ++q) cycles[q] = 0;
    for (size_t g = 0; g < (size_t)kPhaseGroups; ++g)
        for (int q = 0; q < kPhaseCells; ++q) cycles[q] += all[g * kPhaseCells + q];
    if (reset) {
        void *at = nullptr;
        DNATOK_HIP_TRY(hipGetSymbolAddress(&at, HIP_SYMBOL(g_phase_cycles)));
        DNATOK_HIP_TRY(hipMemset(at, 0, all.size() * sizeof(unsigned long long)));
    }
    return DNATOK_OK;
}
#endif
