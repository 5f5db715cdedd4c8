// Beam search over CRF scores, gfx950.
//
// Every chunk is served by two wavefronts of a workgroup.  The loader wave streams the
// rows the search needs (scores[t] as fp16 and bwd[t+1] as fp32) from HBM into an LDS
// ring, several rows ahead; the search wave runs the search with the 32-wide beam
// resident in registers/LDS.  The two communicate through two LDS counters (rows ready /
// rows consumed), so the search never waits on a dependent HBM gather.  A workgroup holds
// two or four chunks, so that its waves spread over the four SIMDs of a compute unit.
//
// Search wave lane layout: lanes 2i and 2i+1 both hold beam element i; lane 2i+h holds
// its step candidates with new base 2h and 2h+1, the even lane also its stay candidate,
// so that lane order is the CPU path's candidate order (steps 4i+b, then stays) and
// ranks are masked bit counts.
// The search reproduces the CPU path (reference src/beam_search.c:117-439) to the
// bit: same fp32 operation order, double-precision log-sum-exp for merges, the
// same cut-off bisection, first-come compaction and final best-to-slot-0 swap.
// Instead of sorting, the cut-off uses wave ballots and population counts, and
// survivors are ranked with ballot prefix counts.
//
// Stay/step merging: a stay of element i merges with the step (j, b_i) whose hash
// crc(hash_j, b_i) equals hash_i.  The 2-bit CRC update is a bijection of the
// 32-bit state, so this is the same as hash_j == crc^-1(hash_i, b_i) =: want_i, the hash
// of the element's sequence without its last base.  Every beam element carries both
// words (a candidate's `want` is its parent's hash, or its parent's `want` for a stay), and
// the element j is found through a hash index in LDS: every live element files
// {hash, generation << 5 | slot} under some bits of its hash, reads its own entry back, and
// looks up the entry filed under the same bits of `want`.  If every element finds its own
// entry intact, all hashes are pairwise distinct and every existing partner is found by
// exactly one probe (the full 32 bits are compared); otherwise (two elements in one
// bucket, about one step in ten; equal hashes, only after a CRC collision) the step
// falls back to comparing `want` with all 32 hashes.
#include <hip/hip_runtime.h>

#include <cfloat>
#include <mutex>
#include <type_traits>

#include "kernels.h"

namespace {

constexpr int kW = OFK_BEAM_WIDTH;
constexpr uint32_t kPoly = 0x82f63b78u;
constexpr uint32_t kSeed = 0x12345678u;

constexpr uint32_t crc_bits(uint32_t crc, uint32_t bits, int n) {
    for (int i = 0; i < n; ++i) {
        const uint32_t feed = (bits ^ crc) & 1u;
        crc >>= 1;
        if (feed) crc ^= kPoly;
        bits >>= 1;
    }
    return crc;
}
// CRC-32C is linear over GF(2): two update steps are (crc >> 2) xor a table entry chosen
// by the two low bits of crc ^ bits, and the entry for 3 is the xor of those for 1 and 2.
constexpr uint32_t kTab1 = crc_bits(1u, 0u, 2);
constexpr uint32_t kTab2 = crc_bits(2u, 0u, 2);
static_assert(crc_bits(3u, 0u, 2) == (kTab1 ^ kTab2), "crc linearity");
static_assert((kTab1 >> 30) == 1u && (kTab2 >> 30) == 2u, "top bits identify the table entry");

__device__ __forceinline__ uint32_t crc_tab(uint32_t x) {
    return ((0u - (x & 1u)) & kTab1) ^ ((0u - ((x >> 1) & 1u)) & kTab2);
}
__device__ __forceinline__ uint32_t crc2(uint32_t crc, uint32_t base) {
    return (crc >> 2) ^ crc_tab((crc ^ base) & 3u);
}
// the hash h with crc2(h, base) == crc
__device__ __forceinline__ uint32_t crc2_inverse(uint32_t crc, uint32_t base) {
    const uint32_t k = crc >> 30;
    return ((crc ^ crc_tab(k)) << 2) | (k ^ base);
}
__device__ __forceinline__ uint32_t crc32_word(uint32_t crc, uint32_t word) {
    for (int i = 0; i < 16; ++i) {
        crc = crc2(crc, word & 3u);
        word >>= 2;
    }
    return crc;
}

template <int CTRL>
__device__ __forceinline__ float dpp(float x) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xF, 0xF, true));
}
__device__ __forceinline__ float lane_f(float x, int lane) {
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(x), lane));
}
__device__ __forceinline__ uint32_t lane_u(uint32_t x, int lane) {
    return (uint32_t)__builtin_amdgcn_readlane((int)x, lane);
}
// Maximum over the wave, every lane active.  The rotate-and-max steps are single DPP
// instructions written out by hand (the compiler's lowering of fmaxf after a DPP move
// adds a move and a canonicalisation per step); each needs two idle cycles after the
// instruction that wrote its source.  The last two steps carry the row maxima across
// rows, so lane 63 ends up with the result.  The inputs are never NaN.
__device__ __forceinline__ float wave_max(float x) {
    asm volatile(
        "s_nop 1\n\t"
        "v_max_f32_dpp %0, %0, %0 row_ror:8 row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\t"
        "v_max_f32_dpp %0, %0, %0 row_ror:4 row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\t"
        "v_max_f32_dpp %0, %0, %0 row_ror:2 row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\t"
        "v_max_f32_dpp %0, %0, %0 row_ror:1 row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\t"
        "v_max_f32_dpp %0, %0, %0 row_bcast:15 row_mask:0xa bank_mask:0xf\n\t"
        "s_nop 1\n\t"
        "v_max_f32_dpp %0, %0, %0 row_bcast:31 row_mask:0xc bank_mask:0xf\n\t"
        "s_nop 1"
        : "+v"(x));
    return lane_f(x, 63);
}
// What a lane will store for its three candidates once their ranks are known, worked out in the
// wait states of the wave maximum: a wave that is alone on its SIMD pays a full issue slot (about
// eight cycles) for every s_nop, so the two idle cycles each rotate-and-max step needs after its
// source was written are filled with instructions that had to be issued anyway.
//   h0 = crc2(hash, b0), h1 = crc2(hash, b0 + 1) = h0 ^ kTab1   (b0 is even)
//   info0 = (lo4 + b0) | from, info1 = info0 | 1, infos = state | from | stay bit
//   rest = candidate score minus its guide term
// The lane maximum (one v_max3) opens the block and the read of lane 63, where the six steps leave
// the wave's maximum, closes it, each with its own wait states filled the same way.
struct NextRecords {
    uint32_t h0, h1, info0, info1, infos;
    float rest0, rest1, rests;
};
__device__ __forceinline__ float wave_max_beside_records(float c0, float c1, float cs, NextRecords &n, uint32_t hash,
                                                         uint32_t b0, uint32_t state, uint32_t from_stay,
                                                         uint32_t lo4b0, uint32_t from, float g0, float g1,
                                                         float gs) {
    uint32_t t0, t1, best;
    float x;
    asm volatile(
        "v_max3_f32 %[x], %[c0], %[c1], %[cs]\n\t"
        "v_xor_b32 %[t0], %[hash], %[b0]\n\t"
        "v_sub_f32 %[r0], %[c0], %[g0]\n\t"
        "v_max_f32_dpp %[x], %[x], %[x] row_ror:8 row_mask:0xf bank_mask:0xf\n\t"
        "v_bfe_i32 %[t1], %[t0], 1, 1\n\t"
        "v_bfe_i32 %[t0], %[t0], 0, 1\n\t"
        "v_max_f32_dpp %[x], %[x], %[x] row_ror:4 row_mask:0xf bank_mask:0xf\n\t"
        "v_and_b32 %[t1], %[tab2], %[t1]\n\t"
        "v_and_b32 %[t0], %[tab1], %[t0]\n\t"
        "v_max_f32_dpp %[x], %[x], %[x] row_ror:2 row_mask:0xf bank_mask:0xf\n\t"
        "v_xor_b32 %[t0], %[t0], %[t1]\n\t"
        "v_lshrrev_b32 %[t1], 2, %[hash]\n\t"
        "v_max_f32_dpp %[x], %[x], %[x] row_ror:1 row_mask:0xf bank_mask:0xf\n\t"
        "v_xor_b32 %[h0], %[t0], %[t1]\n\t"
        "v_sub_f32 %[r1], %[c1], %[g1]\n\t"
        "v_max_f32_dpp %[x], %[x], %[x] row_bcast:15 row_mask:0xa bank_mask:0xf\n\t"
        "v_xor_b32 %[h1], %[tab1], %[h0]\n\t"
        "v_sub_f32 %[rs], %[cs], %[gs]\n\t"
        "v_max_f32_dpp %[x], %[x], %[x] row_bcast:31 row_mask:0xc bank_mask:0xf\n\t"
        "v_or_b32 %[i0], %[lo4b0], %[from]\n\t"
        "v_or_b32 %[is], %[state], %[fromstay]\n\t"
        "v_readlane_b32 %[best], %[x], 63\n\t"
        "v_or_b32 %[i1], 1, %[i0]\n\t"
        "s_nop 0"
        : [x] "=&v"(x), [best] "=&s"(best), [t0] "=&v"(t0), [t1] "=&v"(t1), [h0] "=&v"(n.h0), [h1] "=&v"(n.h1),
          [i0] "=&v"(n.info0), [i1] "=&v"(n.info1), [is] "=&v"(n.infos), [r0] "=&v"(n.rest0), [r1] "=&v"(n.rest1),
          [rs] "=&v"(n.rests)
        : [hash] "v"(hash), [b0] "v"(b0), [tab1] "s"(kTab1), [tab2] "s"(kTab2), [lo4b0] "v"(lo4b0), [from] "v"(from),
          [state] "v"(state), [fromstay] "v"(from_stay), [c0] "v"(c0), [c1] "v"(c1), [cs] "v"(cs), [g0] "v"(g0),
          [g1] "v"(g1), [gs] "v"(gs));
    return __uint_as_float(best);
}
__device__ __forceinline__ int wave_sum_i(int x) {
    x += __builtin_amdgcn_update_dpp(0, x, 0x128, 0xF, 0xF, true);
    x += __builtin_amdgcn_update_dpp(0, x, 0x124, 0xF, 0xF, true);
    x += __builtin_amdgcn_update_dpp(0, x, 0x122, 0xF, 0xF, true);
    x += __builtin_amdgcn_update_dpp(0, x, 0x121, 0xF, 0xF, true);
    return __builtin_amdgcn_readlane(x, 0) + __builtin_amdgcn_readlane(x, 16) +
           __builtin_amdgcn_readlane(x, 32) + __builtin_amdgcn_readlane(x, 48);
}
__device__ __forceinline__ uint64_t ballot(bool p) { return __builtin_amdgcn_ballot_w64(p); }
// per lane: yes where the lane's bit of a wave-wide mask is set, no elsewhere; the mask goes into
// the select as it is (a comparison result the wave already holds in scalar registers).
// The compiler cannot see into these two statements, so it inserts no wait states for them.  None
// are due: a scalar pair written by a vector comparison may be read as the mask of a select or as
// a carry by the next vector instruction (the wait states the architecture asks for after such a
// write concern lane selects of v_readlane/v_writelane, v_div_fmas and memory instructions).  A
// mask that is to be read by v_readlane or as an address goes through an s_mov first.
__device__ __forceinline__ int pick_by_bit(uint64_t mask, int yes, int no) {
    int r;
    asm("v_cndmask_b32_e64 %0, %1, %2, %3" : "=v"(r) : "v"(no), "v"(yes), "s"(mask));
    return r;
}
// x + (the lane's bit of mask), one add-with-carry
__device__ __forceinline__ int add_bit_of(int x, uint64_t mask) {
    int r;
    uint64_t carry;
    asm("v_addc_co_u32_e64 %0, %1, %2, 0, %3" : "=v"(r), "=&s"(carry) : "v"(x), "s"(mask));
    return r;
}
__device__ __forceinline__ int popc64(uint64_t x) { return __builtin_popcountll(x); }
// x + (float)h for the fp16 value h in the low half of a word, in one instruction: v_fma_mix_f32
// converts the half operand on the fly and the product with 1.0 is exact, so the result is the
// correctly rounded fp32 sum, bit for bit what a conversion followed by an addition gives
__device__ __forceinline__ float add_half(uint32_t word, float x) {
    float r;
    asm("v_fma_mix_f32 %0, %1, 1.0, %2 op_sel_hi:[1,0,0]" : "=v"(r) : "v"(word), "v"(x));
    return r;
}
// LDS accesses through a 32-bit LDS address
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
#define LDS_AS __attribute__((address_space(3)))
__device__ __forceinline__ f32x2 lds_load_f2(uint32_t at) { return *(const LDS_AS f32x2 *)(uintptr_t)at; }
__device__ __forceinline__ u32x2 lds_load_u2(uint32_t at) { return *(const LDS_AS u32x2 *)(uintptr_t)at; }
__device__ __forceinline__ float lds_load_f(uint32_t at) { return *(const LDS_AS float *)(uintptr_t)at; }
__device__ __forceinline__ void lds_store_f2(uint32_t at, float a, float b) {
    f32x2 v;
    v.x = a;
    v.y = b;
    *(LDS_AS f32x2 *)(uintptr_t)at = v;
}
__device__ __forceinline__ void lds_store_f(uint32_t at, float a) { *(LDS_AS float *)(uintptr_t)at = a; }
// (x & bits) | base in one instruction
__device__ __forceinline__ uint32_t and_or(uint32_t x, uint32_t bits, uint32_t base) {
    uint32_t r;
    asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(x), "s"(bits), "v"(base));
    return r;
}

__device__ __forceinline__ void wave_fence() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Hand-over of LDS rows between the two waves of a workgroup.  The fences name the
// local address space only: they wait for outstanding LDS operations, not for the
// global loads and stores each wave keeps in flight.
__device__ __forceinline__ void publish(int *flag, int value) {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __hip_atomic_store(flag, value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}
__device__ __forceinline__ int observe(int *flag) {
    const int v = __hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
    return v;
}

// log(e^x + e^y) with the correction evaluated in double and dropped for gaps >= 17
// (reference src/beam_search.c:43-47).  The correction log(1 + e^-gap) comes from a
// piecewise polynomial kept in LDS: a handful of dependent FMAs instead of an exp
// followed by a log, which matters because every merge sits on the search's serial path.
__device__ __forceinline__ float log_sum_exp(float x, float y, const double *table) {
    const float gap = fabsf(x - y);
    const float top = x > y ? x : y;
    int cell = (int)(gap * 4.0f);
    cell = cell < OFK_LSE_CELLS - 1 ? cell : OFK_LSE_CELLS - 1;
    const double *c = table + cell * OFK_LSE_COEFS;
    const double s = __builtin_fma((double)gap, 8.0, -(double)(2 * cell + 1));  // (gap - centre of the cell) * 8, exactly
    double p = c[8];
#pragma unroll
    for (int k = 7; k >= 0; --k) p = __builtin_fma(p, s, c[k]);
    const double corr = gap < 17.0f ? p : 0.0;
    return (float)((double)top + corr);
}

// The same fold from the hardware's fp32 exp2/log2, with the verdict whether its rounded result is
// certain to be the one above.  top + l2 * ln2f (one fused multiply-add, l2 = log2(1 + exp2(-gap c)))
// differs from top + log(1 + e^-gap) by at most, in units of 2^-24:
//   0.72  v_exp_f32 (largest relative error over every input in [-160, 0]: 1.423), times e/(1+e) <= 1/2
//   0.45  the argument of exp2: gap c rounded to fp32 with c = fl(log2 e): 7.3e-8 gap e^-gap <= 2.7e-8
//   1.00  1 + e rounded to fp32
//   1.39  v_log_f32 on [1, 2] (largest absolute error over every input: 1.0 below 2, 2.0 at 2), times ln 2
//   0.08  ln2f against ln 2, the rounding of the residual
// together 3.64; the bound used is 4.0.  (The two hardware figures are measured on the device at
// hand, over every fp32 input of their ranges, by tests/test_gpu_hw_math.py.)  The result is settled when the distance from the
// unrounded sum to the nearer rounding boundary of the result exceeds that bound (the residual of
// the fused multiply-add, taken exactly with a second one).  Half an ulp is read from the exponent
// of the next smaller float, which for a power of two is the binade below, where its nearer
// boundary lies; results that are zero or below 2^-102 in magnitude never count as settled.
__device__ __forceinline__ float log_sum_exp_estimate(float x, float y, bool &settled) {
    const float gap = fabsf(x - y);
    const float top = x > y ? x : y;
    const float e = __builtin_amdgcn_exp2f(gap * -1.44269504088896340736f);
    const float l2 = __builtin_amdgcn_logf(1.0f + e);
    const float kLn2 = 0.69314718055994530942f;
    const float r = __builtin_fmaf(l2, kLn2, top);
    const float rho = __builtin_fmaf(l2, kLn2, -(r - top));
    const uint32_t rb = __float_as_uint(r);
    const float half_ulp = __uint_as_float(((rb & 0x7fffffffu) - ((24u << 23) + 1u)) & 0xff800000u);
    settled = half_ulp - fabsf(rho) > 4.0f * 5.9604644775390625e-8f;
    return r;
}

__device__ __forceinline__ uint32_t float_key(float f) {
    const uint32_t u = __float_as_uint(f);
    return u ^ ((u >> 31) ? 0xFFFFFFFFu : 0x80000000u);
}
__device__ __forceinline__ float key_float(uint32_t k) {
    return __uint_as_float(k ^ ((k >> 31) ? 0x80000000u : 0xFFFFFFFFu));
}

template <int BYTES>
struct Vec;
template <>
struct Vec<4> { typedef uint32_t type; };
template <>
struct Vec<8> { typedef uint32_t type __attribute__((ext_vector_type(2))); };
template <>
struct Vec<16> { typedef uint32_t type __attribute__((ext_vector_type(4))); };

// one wave's share of a row of ROW_BYTES bytes: lane l owns vectors (i*64 + l).  Rows of 256
// and 512 bytes are split into 4- and 8-byte vectors, one per lane; all others into 16-byte
// vectors, of which the last round may cover only the lower lanes (rows of five-column scores
// are 640, 2560 or 10240 bytes).
template <int ROW_BYTES>
struct RowRegs {
    static constexpr int kVec = ROW_BYTES == 256 ? 4 : ROW_BYTES == 512 ? 8 : 16;
    static constexpr int kVecs = ROW_BYTES / kVec;
    static constexpr int kCnt = (kVecs + 63) / 64;
    static_assert(ROW_BYTES % kVec == 0, "rows are whole vectors");
    typedef typename Vec<kVec>::type V;
    V v[kCnt];
    static __device__ __forceinline__ bool mine(int i, int lane) { return (i + 1) * 64 <= kVecs || i * 64 + lane < kVecs; }
    __device__ __forceinline__ void load(const char *row, int lane) {
#pragma unroll
        for (int i = 0; i < kCnt; ++i)
            if (mine(i, lane)) v[i] = *reinterpret_cast<const V *>(row + (size_t)(i * 64 + lane) * kVec);
    }
    __device__ __forceinline__ void store(char *row, int lane) const {
#pragma unroll
        for (int i = 0; i < kCnt; ++i)
            if (mine(i, lane)) *reinterpret_cast<V *>(row + (size_t)(i * 64 + lane) * kVec) = v[i];
    }
};


template <int S>
struct BeamCfg {
    static constexpr int kBits = S == 64 ? 6 : S == 256 ? 8 : 10;
    static constexpr int kLdsRows = S >= 1024 ? 3 : S >= 256 ? 4 : 6;  // LDS ring depth
    static constexpr int kRegRows = S >= 1024 ? 3 : 6;  // rows in flight in registers (3 or 6)
};

// one beam element as handed from one time step to the next: three words of a 16-byte slot, written
// by one 96-bit store (an LDS store costs by its width, whatever the number of enabled lanes)
struct __attribute__((aligned(16))) Elem {
    uint32_t hash;
    float rest;     // candidate score minus the guide term of its state: what the next time step starts from
                    // (at the last time step: the candidate score itself, which picks the best survivor)
    uint32_t info;  // state | prev << 10 | stay << 15: the 16-bit slot the traceback reads
    uint32_t pad;
};

struct BeamShared {
    Elem elem[kW + 64];           // slots 0 .. kW-1; entry kW + lane is lane's dump slot for candidates that are not kept
    float cand[4 * kW + 64];      // scores of the step candidates 4i+b while stays merge into them; then dump slots
    float stay_score[kW];         // only used by the serial replay of merges
    uint32_t claim[4 * kW + 64];  // only used when the hash index was not conclusive: who claimed step candidate 4j+b
    int ready;                    // rows stored by the loader wave
    int consumed;                 // rows the search wave is done with
};

// LDS of one chunk.  Score rows are kept as the caller lays them out: COLS = 4 transitions per
// state, or 5 with an unused blank first.
template <int S, int COLS>
struct BeamRing {
    _Float16 row_s[BeamCfg<S>::kLdsRows][COLS * S];
    float row_b[BeamCfg<S>::kLdsRows][S];
};
// Buckets of the hash index of one chunk (8 bytes each: hash, generation << 5 | slot).  With w
// live elements two of them share a bucket in about w^2 / (2 * buckets) of the time steps.
template <int S, int CPG>
struct BeamIdx {
    static constexpr int kBuckets = (S >= 1024 || CPG > 2) ? 2048 : 4096;
};
template <int S, int COLS>
struct __attribute__((aligned(16))) BeamLds {
    BeamRing<S, COLS> ring;
    BeamShared sh;
    uint2 idx_dump[64];  // where a dead lane files its leftovers instead of a bucket of the index
};
// All LDS of a workgroup, one object: the index tables come first and each is aligned to its
// size, so that a bucket's address is (hash & bits) | table, one instruction.
template <int S, int CPG, int COLS>
struct __attribute__((aligned(BeamIdx<S, CPG>::kBuckets * 8))) BeamGroupLds {
    uint2 idx[CPG][BeamIdx<S, CPG>::kBuckets];
    BeamLds<S, COLS> chunk[CPG];
    double lse[OFK_LSE_DOUBLES];  // coefficient table of the folds, one copy per workgroup
};


// CPG chunks per workgroup.  The waves of a group are dealt round over the four SIMDs of
// its compute unit (wave k and wave k + 4 share one), while two-wave groups were measured
// to pile onto two SIMDs.  With two chunks a group is four waves, two of them searching;
// with four chunks it is eight waves and every SIMD holds exactly one search wave and one
// loader, which is what a batch of more than two chunks per compute unit needs.
template <int S, int CPG, int COLS>
__global__ __launch_bounds__(128 * CPG) void beam_kernel(const _Float16 *__restrict__ scores,
                                                   const float *__restrict__ bwd,
                                                   ofk_beam_slot_t *__restrict__ beam,
                                                   int32_t *__restrict__ states, uint8_t *__restrict__ moves,
                                                   int T, int N, float log_cut, float stay, int flags,
                                                   const double *__restrict__ lse_table) {
    using Cfg = BeamCfg<S>;
    constexpr int BITS = Cfg::kBits;
    constexpr int LR = Cfg::kLdsRows;
    constexpr int RR = Cfg::kRegRows;

    constexpr int kGroupChunks = CPG;
    __shared__ BeamGroupLds<S, CPG, COLS> all;
    auto &lds = all.chunk;
    auto &lse = all.lse;

    // waves 0 .. kGroupChunks-1 search, the others load; wave k and wave k + kGroupChunks share a chunk
    const int wave = (int)(threadIdx.x >> 6);
    const int member = wave % kGroupChunks;
    const int n = blockIdx.x * kGroupChunks + member;
    const int lane = threadIdx.x & 63;
    auto &row_s = lds[member].ring.row_s;
    auto &row_b = lds[member].ring.row_b;
    BeamShared &sh = lds[member].sh;
    const size_t row_stride = (size_t)N * COLS * S;
    const _Float16 *sc_n = scores + (size_t)n * COLS * S;
    const float *bw_n = bwd + (size_t)n * (size_t)(T + 1) * S;

    if (wave < kGroupChunks && lane == 0) {
        sh.ready = 0;
        sh.consumed = 0;
    }
    for (int x = (int)threadIdx.x; x < OFK_LSE_DOUBLES; x += 128 * CPG) lse[x] = lse_table[x];
    // the hash index starts empty: no entry may look like one of a real generation (tags start at 1 << 5)
    for (int x = (int)threadIdx.x; x < kGroupChunks * BeamIdx<S, CPG>::kBuckets; x += 128 * CPG) (&all.idx[0][0])[x] = make_uint2(0u, 0u);
    __syncthreads();
    if (n >= N) return;  // odd batch: the last group has one chunk

    if (wave >= kGroupChunks) {
        // ---- loader wave: row t = (scores[t], bwd[t+1]) into ring slot t % LR ----
        // The ring is spelled out as named registers (not an array indexed by a loop that
        // also contains the spin wait) so that every row stays in VGPRs.
        RowRegs<2 * COLS * S> s0, s1, s2, s3, s4, s5;
        RowRegs<4 * S> g0, g1, g2, g3, g4, g5;
        auto fetch = [&](RowRegs<2 * COLS * S> &rs, RowRegs<4 * S> &rb, int t) {
            if (t < T) {
                rs.load(reinterpret_cast<const char *>(sc_n + (size_t)t * row_stride), lane);
                rb.load(reinterpret_cast<const char *>(bw_n + (size_t)(t + 1) * S), lane);
            }
        };
        auto hand_over = [&](RowRegs<2 * COLS * S> &rs, RowRegs<4 * S> &rb, int t) {
            if (t < T) {
                // the ring is full most of the time (a search step takes about 3000 cycles): poll
                // seldom, the rows in registers and in the ring leave ample slack for waking up late
                while (t - observe(&sh.consumed) >= LR) __builtin_amdgcn_s_sleep(8);
                const int slot = t % LR;
                rs.store(reinterpret_cast<char *>(row_s[slot]), lane);
                rb.store(reinterpret_cast<char *>(row_b[slot]), lane);
                fetch(rs, rb, t + RR);
                publish(&sh.ready, t + 1);
            }
        };
        fetch(s0, g0, 0);
        fetch(s1, g1, 1);
        fetch(s2, g2, 2);
        if constexpr (RR == 6) {
            fetch(s3, g3, 3);
            fetch(s4, g4, 4);
            fetch(s5, g5, 5);
        }
        for (int t0 = 0; t0 < T; t0 += RR) {
            hand_over(s0, g0, t0);
            hand_over(s1, g1, t0 + 1);
            hand_over(s2, g2, t0 + 2);
            if constexpr (RR == 6) {
                hand_over(s3, g3, t0 + 3);
                hand_over(s4, g4, t0 + 4);
                hand_over(s5, g5, t0 + 5);
            }
        }
        return;
    }

    // ---- search wave ----
    const int i = lane >> 1;  // lanes 2i and 2i+1 hold element i; candidate order is lane order
    const int h = lane & 1;
    constexpr int kBuckets = BeamIdx<S, CPG>::kBuckets;
    constexpr uint32_t kBucketBits = (uint32_t)(kBuckets - 1) << 3;  // hash bits that address an 8-byte bucket
    typedef __attribute__((address_space(3))) uint32_t lds_u32;
    // LDS addresses of this chunk's index table (a multiple of its size) and of this lane's spare entry
    const uint32_t idx_base = (uint32_t)(uintptr_t)(lds_u32 *)&all.idx[member][0].x;
    const uint32_t idx_dump = (uint32_t)(uintptr_t)(lds_u32 *)&lds[member].idx_dump[lane].x;

    // seeding: the 32 best states of bwd[0] in ascending state order (src/beam_search.c:151-175)
    {
        constexpr int PER = S / 64;
        float v[PER];
        uint32_t key[PER];
#pragma unroll
        for (int j = 0; j < PER; ++j) {
            v[j] = bw_n[j * 64 + lane];
            key[j] = float_key(v[j]);
        }
        uint32_t prefix = 0;  // largest K with #{key >= K} >= 32, i.e. the 32nd largest value
        for (int bit = 31; bit >= 0; --bit) {
            const uint32_t trial = prefix | (1u << bit);
            int c = 0;
#pragma unroll
            for (int j = 0; j < PER; ++j) c += key[j] >= trial ? 1 : 0;
            if (wave_sum_i(c) >= kW) prefix = trial;
        }
        const float thr = key_float(prefix);
        if (lane < kW) sh.elem[lane] = Elem{0u, 0.f, 0u, 0u};
        wave_fence();
        int taken = 0;
#pragma unroll
        for (int j = 0; j < PER; ++j) {
            const bool ok = v[j] >= thr;
            const uint64_t m = ballot(ok);
            const int rank = taken + popc64(m & (((uint64_t)1 << lane) - 1));
            if (ok && rank < kW) {
                const uint32_t s = (uint32_t)(j * 64 + lane);
                // flags bit 1 (tests): seeds that agree in their low four state bits share a hash
                const uint32_t hs = crc32_word(kSeed, (flags & 2) ? (s & 15u) : s);
                sh.elem[rank] = Elem{hs, 0.f, s, 0u};
            }
            taken += popc64(m);
        }
        wave_fence();
    }
    uint32_t hash, want, info;  // want: the hash of the sequence without its last base, what a partner's hash has to equal
    float score;
    {
        const Elem e = sh.elem[i];
        hash = e.hash;
        info = e.info;
        score = e.rest;
    }
    int state = (int)(info & 1023u);
    want = crc2_inverse(hash, (uint32_t)state & 3u);
    int w = kW;
    ofk_beam_slot_t *bv = beam + (size_t)n * (size_t)(T + 1) * kW;
    bv[i] = (ofk_beam_slot_t)state;

    // The search is a chain of dependent short instructions; when it shares a SIMD with
    // throughput-bound waves (the forward scan runs at the same time) it should win the
    // issue arbitration.
    __builtin_amdgcn_s_setprio(3);
    // Only the even lane of a pair carries the element's stay.  The odd lane adds -FLT_MAX instead of
    // the stay score, so that its stay candidate is -FLT_MAX (or -inf once the element is dead):
    // it never passes a cut and never wins a maximum, without a select in every time step.
    const float stay_h = h == 0 ? stay : -FLT_MAX;
    const uint32_t from = (uint32_t)i << 10, from_stay = from | (1u << 15);  // the element's index as "prev" of its candidates
    int rows_ready = 0;  // last value seen of the loader's counter; it is usually several rows ahead
    const int b0 = 2 * h;
    const uint32_t cand_base = (uint32_t)(uintptr_t)(lds_u32 *)&sh.cand[0];
    const uint32_t cand_mine = cand_base + 8u * (uint32_t)lane;           // candidates 4i+b0, 4i+b0+1
    const uint32_t cand_dump = cand_base + 4u * (uint32_t)(4 * kW + lane);  // where a stay without a partner writes
    // What a time step reads from LDS depends only on the beam it starts from, so it is
    // fetched as soon as that beam is known (at the end of the previous step): the row
    // entries of the lane's candidates, and the hash index: the element's own entry goes in, is
    // read back, and the entry filed under `want` is read.
    uint32_t r0h, r1h;  // fp16 scores of the lane's two step candidates, each in the low half of a word
    f32x2 g01;
    float gst;
    u32x2 probe;     // index entry found under `want`
    uint32_t mine_back;  // tag found under the element's own hash
    uint32_t tagv;   // generation << 5 | slot of this element (generation = time step + 1)
    uint64_t vm = ~0ull;  // lanes of live elements
    // ring addresses: the same in every lane, kept in scalar registers
    const uint32_t ring_s = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uintptr_t)(lds_u32 *)&row_s[0][0]);
    const uint32_t ring_b = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uintptr_t)(lds_u32 *)&row_b[0][0]);
    auto fetch_row = [&](int tt) {
        while (__builtin_expect(rows_ready <= tt, 0)) {  // the counter is one LDS word: the same value in every lane
            rows_ready = __builtin_amdgcn_readfirstlane(observe(&sh.ready));
            if (rows_ready <= tt) __builtin_amdgcn_s_sleep(1);
        }
        const uint32_t slot = (uint32_t)tt % (uint32_t)LR;
        const uint32_t rs = ring_s + slot * (uint32_t)(2 * COLS * S);  // scalar
        const uint32_t rb = ring_b + slot * (uint32_t)(4 * S);
        // scores of the candidates with bases b0, b0 + 1: rs[COLS * (lo4 + b0 + {0,1}) + (COLS - 4) + top];
        // guide terms rb[lo4 + b0 + {0,1}] and rb[state]
        const uint32_t st4 = (uint32_t)state << 2;
        const uint32_t cand = and_or(st4, (uint32_t)(S - 1), (uint32_t)b0);  // lo4 + b0
        const uint32_t top = ((uint32_t)state >> (BITS - 2)) << 1;  // byte offset of the dropped base's column
        uint32_t at_s;
        if constexpr (COLS == 4) at_s = (cand << 3) + rs;
        else at_s = cand * 10u + rs;
        at_s += top;
        typedef __attribute__((address_space(3))) uint16_t lds_u16;
        r0h = *(const lds_u16 *)(uintptr_t)(at_s + 2u * (COLS - 4));
        r1h = *(const lds_u16 *)(uintptr_t)(at_s + 2u * (COLS - 4) + 2u * COLS);
        g01 = lds_load_f2((cand << 2) + rb);
        gst = lds_load_f(st4 + rb);
        // hash index of the beam this step starts from; dead lanes file their leftovers apart
        tagv = ((uint32_t)(tt + 1) << 5) | (uint32_t)i;
        const uint32_t own = (uint32_t)pick_by_bit(vm, (int)and_or(hash, kBucketBits, idx_base), (int)idx_dump);
        const uint32_t wanted = and_or(want, kBucketBits, idx_base);
        lds_u32 *own_p = (lds_u32 *)(uintptr_t)own;
        own_p[0] = hash;
        own_p[1] = tagv;
        wave_fence();  // one wave's LDS operations are carried out in order: the reads below see every lane's entry
        probe = lds_load_u2(wanted);
        mine_back = own_p[1];
    };
    fetch_row(0);
    const uint64_t replay_all = (flags & 1) ? ~0ull : 0ull;
    // One time step.  The last one (LAST) differs in what it hands on (nothing is fetched for a next
    // step, the best survivor goes to slot 0) and is compiled apart, so that the others carry no
    // test for it.
    auto step = [&](const int t, auto last_tag) {
        constexpr bool LAST = decltype(last_tag)::value;
        const uint64_t vs = vm & 0x5555555555555555ull;  // the stay candidates sit on the even lanes
        const int lo4 = (state << 2) & (S - 1);
        // (score + transition) + guide, the CPU path's order of additions; the fp16 transition is
        // converted inside the first addition
        float c0 = add_half(r0h, score) + g01.x;
        float c1 = add_half(r1h, score) + g01.y;
        float cs = (score + stay_h) + gst;
        publish(&sh.consumed, t + 1);  // everything this step needs of row t is in registers
        const uint32_t gen = (uint32_t)(t + 1) << 5;

        // which previous element j has hash_j == want_i: off the index if every live element found its
        // own entry intact, else by comparing with every hash
        uint32_t j;
        uint64_t mine_mask;  // live even lanes whose stay has a partner
        const uint64_t stale = (ballot(mine_back != tagv) & vm) | replay_all;
        if (__builtin_expect(stale == 0, 1)) {
            const uint32_t d = probe.y - gen;  // below 32: an entry of this generation, and d is its slot
            mine_mask = ballot(d < 32u) & ballot(probe.x == want) & vs;
            j = d & 31u;
        } else {
            // Two live elements in one bucket (or with one hash).  Bit k of m says whether hash k of this
            // half of the beam equals `want`: each comparison is shifted into an accumulator with an
            // add-with-carry (a = 2a + equal), two accumulators so that no instruction waits for the one
            // before it.
            uint32_t hq[16];
#pragma unroll
            for (int k = 0; k < 16; ++k) hq[k] = sh.elem[16 * h + k].hash;
            uint32_t lo8, hi8;
            {
                uint64_t e0, e1, e2, e3, f0, f1, f2, f3, carry;
                asm("v_cmp_eq_u32_e64 %[e3], %[w], %[x3]\n\t"
                    "v_cmp_eq_u32_e64 %[f3], %[w], %[y3]\n\t"
                    "v_cmp_eq_u32_e64 %[e2], %[w], %[x2]\n\t"
                    "v_cmp_eq_u32_e64 %[f2], %[w], %[y2]\n\t"
                    "v_cmp_eq_u32_e64 %[e1], %[w], %[x1]\n\t"
                    "v_cmp_eq_u32_e64 %[f1], %[w], %[y1]\n\t"
                    "v_cmp_eq_u32_e64 %[e0], %[w], %[x0]\n\t"
                    "v_cmp_eq_u32_e64 %[f0], %[w], %[y0]\n\t"
                    "v_addc_co_u32_e64 %[ax], %[c], 0, 0, %[e3]\n\t"
                    "v_addc_co_u32_e64 %[ay], %[c], 0, 0, %[f3]\n\t"
                    "v_addc_co_u32_e64 %[ax], %[c], %[ax], %[ax], %[e2]\n\t"
                    "v_addc_co_u32_e64 %[ay], %[c], %[ay], %[ay], %[f2]\n\t"
                    "v_addc_co_u32_e64 %[ax], %[c], %[ax], %[ax], %[e1]\n\t"
                    "v_addc_co_u32_e64 %[ay], %[c], %[ay], %[ay], %[f1]\n\t"
                    "v_addc_co_u32_e64 %[ax], %[c], %[ax], %[ax], %[e0]\n\t"
                    "v_addc_co_u32_e64 %[ay], %[c], %[ay], %[ay], %[f0]"
                    : [ax] "=&v"(lo8), [ay] "=&v"(hi8), [e0] "=&s"(e0), [e1] "=&s"(e1), [e2] "=&s"(e2),
                      [e3] "=&s"(e3), [f0] "=&s"(f0), [f1] "=&s"(f1), [f2] "=&s"(f2), [f3] "=&s"(f3),
                      [c] "=&s"(carry)
                    : [w] "v"(want), [x0] "v"(hq[4]), [x1] "v"(hq[5]), [x2] "v"(hq[6]), [x3] "v"(hq[7]),
                      [y0] "v"(hq[12]), [y1] "v"(hq[13]), [y2] "v"(hq[14]), [y3] "v"(hq[15]));
                asm("v_cmp_eq_u32_e64 %[e3], %[w], %[x3]\n\t"
                    "v_cmp_eq_u32_e64 %[f3], %[w], %[y3]\n\t"
                    "v_cmp_eq_u32_e64 %[e2], %[w], %[x2]\n\t"
                    "v_cmp_eq_u32_e64 %[f2], %[w], %[y2]\n\t"
                    "v_cmp_eq_u32_e64 %[e1], %[w], %[x1]\n\t"
                    "v_cmp_eq_u32_e64 %[f1], %[w], %[y1]\n\t"
                    "v_cmp_eq_u32_e64 %[e0], %[w], %[x0]\n\t"
                    "v_cmp_eq_u32_e64 %[f0], %[w], %[y0]\n\t"
                    "v_addc_co_u32_e64 %[ax], %[c], %[ax], %[ax], %[e3]\n\t"
                    "v_addc_co_u32_e64 %[ay], %[c], %[ay], %[ay], %[f3]\n\t"
                    "v_addc_co_u32_e64 %[ax], %[c], %[ax], %[ax], %[e2]\n\t"
                    "v_addc_co_u32_e64 %[ay], %[c], %[ay], %[ay], %[f2]\n\t"
                    "v_addc_co_u32_e64 %[ax], %[c], %[ax], %[ax], %[e1]\n\t"
                    "v_addc_co_u32_e64 %[ay], %[c], %[ay], %[ay], %[f1]\n\t"
                    "v_addc_co_u32_e64 %[ax], %[c], %[ax], %[ax], %[e0]\n\t"
                    "v_addc_co_u32_e64 %[ay], %[c], %[ay], %[ay], %[f0]"
                    : [ax] "+v"(lo8), [ay] "+v"(hi8), [e0] "=&s"(e0), [e1] "=&s"(e1), [e2] "=&s"(e2),
                      [e3] "=&s"(e3), [f0] "=&s"(f0), [f1] "=&s"(f1), [f2] "=&s"(f2), [f3] "=&s"(f3),
                      [c] "=&s"(carry)
                    : [w] "v"(want), [x0] "v"(hq[0]), [x1] "v"(hq[1]), [x2] "v"(hq[2]), [x3] "v"(hq[3]),
                      [y0] "v"(hq[8]), [y1] "v"(hq[9]), [y2] "v"(hq[10]), [y3] "v"(hq[11]));
            }
            uint32_t m = lo8 | (hi8 << 8);
            m <<= 16 * h;
            // the two lanes of an element looked at 16 hashes each and join their masks
            m |= (uint32_t)__builtin_amdgcn_update_dpp(0, (int)m, 0xB1 /* quad_perm:[1,0,3,2] */, 0xF, 0xF, true);
            const uint32_t live = w >= 32 ? 0xFFFFFFFFu : ((1u << w) - 1u);
            const uint32_t match = m & live;
            mine_mask = ballot(match != 0u) & vs;
            j = (uint32_t)__builtin_ctz(match | 0x80000000u) & 31u;
            // Merges in parallel need every stay to have one partner and every step candidate one claimant.
            // Otherwise (only possible after a CRC collision; flags bit 0 forces it) the merges are
            // replayed one by one in the CPU path's order, from the scores as they were before any merge.
            const uint32_t claim_at = (uint32_t)pick_by_bit(mine_mask, (int)(4u * j + ((uint32_t)state & 3u)), 4 * kW + lane);
            sh.claim[claim_at] = (uint32_t)i;
            wave_fence();
            const uint32_t claimed = sh.claim[claim_at];
            const uint32_t odd = (match & (match - 1u)) | (claimed ^ (uint32_t)i);
            if ((ballot(odd != 0u) & mine_mask) != 0 || (flags & 1)) {
                lds_store_f2(cand_mine, c0, c1);
                if (h == 0) sh.stay_score[i] = cs;
                wave_fence();
                if (lane == 0) {
                    for (int a = 0; a < w; ++a) {
                        const uint32_t ha = sh.elem[a].hash;
                        const uint32_t base = sh.elem[a].info & 3u;
                        for (int b = 0; b < w; ++b) {
                            if (crc2(sh.elem[b].hash, base) != ha) continue;
                            float *st = &sh.cand[4 * b + (int)base];
                            const float both = log_sum_exp(sh.stay_score[a], *st, lse);
                            if (sh.stay_score[a] > *st) {
                                sh.stay_score[a] = both;
                                *st = -FLT_MAX;
                            } else {
                                *st = both;
                                sh.stay_score[a] = -FLT_MAX;
                            }
                        }
                    }
                }
                wave_fence();
                const f32x2 c01 = lds_load_f2(cand_mine);
                c0 = c01.x;
                c1 = c01.y;
                if (h == 0) cs = sh.stay_score[i];
                mine_mask = 0;
            }
        }

        // merge stays with the step spelling the same sequence (src/beam_search.c:281-316).  Every lane
        // files its two step candidates; a stay with a partner reads the partner's score, folds the
        // two, keeps its half of the outcome and overwrites the partner with the other half; every
        // lane reads its step candidates back.  Lanes without a merge go through the same
        // instructions with whatever their registers hold and a dump slot as target: no exec
        // masking on the way.  Conditions are kept as wave-wide masks in scalar registers and combined
        // there; a select takes its mask as it is.
        if (__builtin_expect(mine_mask != 0, 1)) {
            lds_store_f2(cand_mine, c0, c1);
            uint32_t at;  // the partner: step candidate 4j + last base of this element
            asm("v_lshl_add_u32 %0, %1, 4, %2" : "=v"(at) : "v"(j), "v"(cand_base + (((uint32_t)state & 3u) << 2)));
            wave_fence();
            const float other = lds_load_f(at);
            const uint64_t stay_wins = ballot(cs > other) & mine_mask;
            const uint64_t step_wins = mine_mask & ~stay_wins;
            // the fold from hardware exp/log where that provably rounds like the CPU path's double
            // arithmetic (all but a few merges in a thousand at usual score magnitudes)
            bool settled;
            float folded = log_sum_exp_estimate(cs, other, settled);
            if (__builtin_expect((ballot(!settled) & mine_mask) != 0, 0)) folded = log_sum_exp(cs, other, lse);
            const uint32_t target = (uint32_t)pick_by_bit(mine_mask, (int)at, (int)cand_dump);
            lds_store_f(target, __int_as_float(pick_by_bit(step_wins, __float_as_int(folded), __float_as_int(-FLT_MAX))));
            cs = __int_as_float(pick_by_bit(stay_wins, __float_as_int(folded), __float_as_int(cs)));
            cs = __int_as_float(pick_by_bit(step_wins, __float_as_int(-FLT_MAX), __float_as_int(cs)));
            wave_fence();
            const f32x2 c01 = lds_load_f2(cand_mine);
            c0 = c01.x;
            c1 = c01.y;
        }

        // cut-off (src/beam_search.c:320-381)
        // Dead lanes carry -FLT_MAX as their score, which absorbs whatever is added: their candidates
        // are -FLT_MAX exactly (the stay of an odd lane: -FLT_MAX or -inf, see stay_h).
        NextRecords next;
        const float best = wave_max_beside_records(c0, c1, cs, next, hash, (uint32_t)b0, (uint32_t)state, from_stay,
                                                   (uint32_t)(lo4 + b0), from, g01.x, g01.y, gst);

        float cut = best - log_cut;  // may be -FLT_MAX (no cut at all): mask the dead lanes
        uint64_t k0 = ballot(c0 >= cut) & vm, k1 = ballot(c1 >= cut) & vm, ks = ballot(cs >= cut) & vs;
        int kept = popc64(k0) + popc64(k1) + popc64(ks);
        bool overfull = false;  // more candidates than the width pass the final cut (the same in every lane)
        if (__builtin_expect(kept > kW, 1)) {
            // Bisection between the cut and the best score.  Every cut tried in here lies above
            // (-FLT_MAX + best) / 2, so dead lanes and dropped candidates never pass and the
            // ballots need no mask.  (lo + hi) / 2 is the CPU path's (cut + hi) / 2 or
            // (cut + lo) / 2: one of the two bounds is the cut just tried.
            float lo = cut, hi = best;
            bool found = false;
#pragma unroll
            for (int guess = 2; guess < 10; ++guess) {
                const bool up = kept > kW;
                lo = up ? cut : lo;
                hi = up ? hi : cut;
                cut = (lo + hi) / 2.0f;
                k0 = ballot(c0 >= cut);
                k1 = ballot(c1 >= cut);
                ks = ballot(cs >= cut);
                kept = popc64(k0) + popc64(k1) + popc64(ks);
                if ((unsigned)(kept - (kW * 8) / 10) <= (unsigned)(kW - (kW * 8) / 10)) {  // 25..32 kept
                    found = true;
                    break;
                }
            }
            if (__builtin_expect(!found, 0)) {
                // The tenth guess: the CPU path moves its bounds once more, tries a cut whose count it
                // never looks at, and settles for the upper bound, whatever that keeps.
                hi = kept > kW ? hi : cut;
                cut = hi;
                k0 = ballot(c0 >= cut);
                k1 = ballot(c1 >= cut);
                ks = ballot(cs >= cut);
                kept = popc64(k0) + popc64(k1) + popc64(ks);
                overfull = kept > kW;
                if (overfull) kept = kW;
            }
        }

        // survivors in candidate order: steps (i, b) by i then b, then stays by i
        {
            // The masks may come straight from vector compares; the selects below are written as
            // instructions and read them as scalar operands, which a vector instruction may do only two
            // instructions after a vector instruction wrote them: scalar copies are safe to read at once.
            asm volatile("s_mov_b64 %0, %0\n\ts_mov_b64 %1, %1\n\ts_mov_b64 %2, %2" : "+s"(k0), "+s"(k1), "+s"(ks));
            // kept candidates on lower lanes: masked bit counts
            auto lower = [&](uint64_t mask, int start) {
                return (int)__builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32),
                                                      __builtin_amdgcn_mbcnt_lo((uint32_t)mask, (uint32_t)start));
            };
            // k0, k1 and ks hold this lane's own verdicts at its bit (dead lanes and the stays of the odd
            // lanes never pass): the masks select directly, nothing is compared again
            const int rank0 = lower(k1, lower(k0, 0));
            const int rank1 = add_bit_of(rank0, k0);
            const int ranks = lower(ks, popc64(k0) + popc64(k1));
            // every lane stores all three of its candidates, the ones that are dropped into its own dump
            // slot: no exec masking on the path from the cut-off to the next beam.  Kept candidates
            // beyond the width exist only after the ten-guess exit of the bisection; a branch that is
            // almost never taken sends them to the dump slot as well.
            const int dump = kW + lane;
            int slot0 = pick_by_bit(k0, rank0, dump);
            int slot1 = pick_by_bit(k1, rank1, dump);
            int slots = pick_by_bit(ks, ranks, dump);
            if (__builtin_expect(overfull, 0)) {
                asm volatile("");  // keeps this a branch instead of three selects on every step
                slot0 = slot0 >= kW ? dump : slot0;
                slot1 = slot1 >= kW ? dump : slot1;
                slots = slots >= kW ? dump : slots;
            }
            if constexpr (LAST) {
                // the last beam is ranked by its candidate scores (src/beam_search.c:398-414)
                next.rest0 = c0;
                next.rest1 = c1;
                next.rests = cs;
            }
            const uint32_t elem_base = (uint32_t)(uintptr_t)(lds_u32 *)&sh.elem[0].hash;
            typedef uint32_t u32x3 __attribute__((ext_vector_type(3)));
            auto put = [&](int slot, uint32_t hsh, uint32_t inf, float rst) {
                uint32_t at_elem;
                asm("v_lshl_add_u32 %0, %1, 4, %2" : "=v"(at_elem) : "v"(slot), "v"(elem_base));
                u32x3 rec;
                rec.x = hsh;
                rec.y = __float_as_uint(rst);
                rec.z = inf;
                *(LDS_AS u32x3 *)(uintptr_t)at_elem = rec;
            };
            put(slot0, next.h0, next.info0, next.rest0);
            put(slot1, next.h1, next.info1, next.rest1);
            put(slots, hash, next.infos, next.rests);
            wave_fence();
        }
        w = kept;
        vm = w > 0 ? ~0ull >> (64 - 2 * w) : 0ull;  // (the best candidate is always kept: w is zero only after NaN scores)
        // every lane reads its slot; slots past the new width hold leftovers: they count as dead through
        // their score and persist as zero, which is what the CPU path's untouched slots hold (a beam
        // cut below 1 empties the beam, and the traceback then walks such slots)
        {
            typedef uint32_t u32x3 __attribute__((ext_vector_type(3)));
            const u32x3 e = *(const LDS_AS u32x3 *)(uintptr_t)((uint32_t)(uintptr_t)(lds_u32 *)&sh.elem[0].hash + 16u * (uint32_t)i);
            hash = e.x;
            info = (uint32_t)pick_by_bit(vm, (int)e.z, 0);
            score = __int_as_float(pick_by_bit(vm, __float_as_int(__uint_as_float(e.y)), __float_as_int(-FLT_MAX)));
        }
        state = (int)(info & 1023u);
        want = crc2_inverse(hash, (uint32_t)state & 3u);
        if constexpr (!LAST) fetch_row(t + 1);

        // last block: the best survivor goes to slot 0 (src/beam_search.c:398-414)
        if constexpr (LAST) {
            const bool in = i < w;
            const float top_score = wave_max(score);
            const uint64_t at = ballot(in && h == 0 && score == top_score);
            const int arg_lane = (top_score > -FLT_MAX && at != 0) ? __builtin_ctzll(at) : 0;  // an even lane
            const int arg = arg_lane >> 1;
            if (arg != 0) {
                const uint32_t in0 = lane_u(info, 0), ina = lane_u(info, arg_lane);
                if (i == 0) info = ina;
                if (i == arg) info = in0;
            }
        }

        // persist the slot (src/beam_search.c:417-427); the guide term was dropped again by the lane
        // that held the candidate, which had the term at hand.  Both halves hold the same element
        // and store the same slot; slots past the width are never followed by the traceback
        bv[(size_t)(t + 1) * kW + i] = (ofk_beam_slot_t)info;
    };
    for (int t = 0; t < T - 1; ++t) step(t, std::false_type{});
    step(T - 1, std::true_type{});

    // ---- traceback from slot 0 of the last block (src/beam_search.c:432-439) ----
    // Followed one row at a time the walk is a chain of T dependent LDS reads.  It is done per block
    // of 128 rows instead, staged in LDS (in the memory of the hash index, which is dead now), in two
    // passes.  Pass 1 walks the block's eight sub-blocks of 16 rows at the same time, each from all
    // 32 slots it could be entered through (lanes 0..31 the four newer sub-blocks, lanes 32..63 the
    // four older ones): where every entry leaves its sub-block.  Eight lane reads then thread the
    // real entry through the block.  Pass 2 walks the eight sub-blocks again, each from its real
    // entry (eight lanes per sub-block, lane q keeping rows 2q and 2q+1 of the walk), and the
    // wave stores 128 states and moves side by side.  Rows that a block lacks at its old end are
    // staged as slots that point at themselves.  The next block's slots travel from global memory
    // while a block is walked.
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    {
        constexpr int RB = 128;  // rows per block
        static_assert(2 * RB * kW * (int)sizeof(ofk_beam_slot_t) <= BeamIdx<S, CPG>::kBuckets * 8, "two blocks fit the index");
        int32_t *st_out = states + (size_t)n * T;
        uint8_t *mv_out = moves + (size_t)n * T;
        const uint32_t buf0 = idx_base;  // two buffers of RB rows of 64 bytes, row 127 the newest of a block
        typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
        u32x4 pre[8];  // a block on its way from global memory: 16-byte piece 64 k + lane in pre[k]
        // block b covers rows hi - rows + 1 .. hi with hi = T - RB b; piece x of the buffer holds
        // row x / 4 - (RB - rows) of those, or slots pointing at themselves before that
        auto load_block = [&](int hi) {
            const int rows = hi < RB ? hi : RB;
            const u32x4 *src = reinterpret_cast<const u32x4 *>(bv + (size_t)(hi - rows + 1) * kW);
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                const int x = 64 * k + lane - 4 * (RB - rows);
                pre[k] = src[x > 0 ? x : 0];  // every lane loads (pieces before the block's first are not used)
            }
        };
        auto store_block = [&](int hi, uint32_t buf) {
            const int rows = hi < RB ? hi : RB;
            const uint32_t c8 = (uint32_t)(lane & 3) * 8u;  // first of the eight slots of an identity piece
            u32x4 self;
            self.x = ((c8 + 0u) << 10) | ((c8 + 1u) << 26);
            self.y = ((c8 + 2u) << 10) | ((c8 + 3u) << 26);
            self.z = ((c8 + 4u) << 10) | ((c8 + 5u) << 26);
            self.w = ((c8 + 6u) << 10) | ((c8 + 7u) << 26);
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                const int x = 64 * k + lane - 4 * (RB - rows);
                *(LDS_AS u32x4 *)(uintptr_t)(buf + 16u * (uint32_t)(64 * k + lane)) = x >= 0 ? pre[k] : self;
            }
        };
        auto slot_at = [&](uint32_t row_base, uint32_t cur, int row) {  // slot `cur` of row `row` above row_base
            uint32_t at;
            asm("v_lshl_add_u32 %0, %1, 1, %2" : "=v"(at) : "v"(cur), "v"(row_base));
            return (uint32_t) * (const LDS_AS uint16_t *)(uintptr_t)(at + 64u * (uint32_t)row);
        };
        uint32_t cursor = 0;  // slot through which the walk enters the block: the same in every lane
        load_block(T);
        store_block(T, buf0);
        int blk = 0;
        for (int hi = T; hi > 0; hi -= RB, ++blk) {
            const int rows = hi < RB ? hi : RB;
            const uint32_t buf = buf0 + (uint32_t)(blk & 1) * (uint32_t)(RB * 64);
            if (hi > RB) load_block(hi - RB);
            wave_fence();
            // pass 1: sub-block s = 4 (lane / 32) + k covers buffer rows 127 - 16 s down to 112 - 16 s
            uint32_t cur[4];
            const uint32_t low1 = buf + 64u * (uint32_t)(112 - 64 * (lane >> 5));  // oldest row of this lane's sub-block k = 0
#pragma unroll
            for (int k = 0; k < 4; ++k) cur[k] = (uint32_t)lane & 31u;
#pragma unroll
            for (int r = 15; r >= 0; --r) {
                uint32_t e[4];
#pragma unroll
                for (int k = 0; k < 4; ++k) e[k] = slot_at(low1 - (uint32_t)(16 * 64 * k), cur[k], r);
#pragma unroll
                for (int k = 0; k < 4; ++k) cur[k] = (e[k] >> 10) & 31u;
            }
            // the real entry of every sub-block
            uint32_t enter[8];
#pragma unroll
            for (int sb = 0; sb < 8; ++sb) {
                enter[sb] = cursor;
                cursor = (uint32_t)__builtin_amdgcn_readlane((int)cur[sb & 3], (int)(cursor + 32u * (uint32_t)(sb >> 2)));
            }
            // pass 2: lanes 8 s .. 8 s + 7 walk sub-block s from its real entry; lane q keeps rows 2q, 2q+1 of the walk
            const int sb2 = lane >> 3, q = lane & 7;
            uint32_t walk = enter[0];
#pragma unroll
            for (int sb = 1; sb < 8; ++sb) walk = sb2 == sb ? enter[sb] : walk;
            const uint32_t low2 = buf + 64u * (uint32_t)(112 - 16 * sb2);
            uint32_t newer = 0, older = 0;
#pragma unroll
            for (int r = 15; r >= 0; --r) {
                const uint32_t e = slot_at(low2, walk, r);
                if (r & 1) newer = q == (15 - r) / 2 ? e : newer;
                else older = q == (15 - r) / 2 ? e : older;
                walk = (e >> 10) & 31u;
            }
            // the next block goes into the other buffer before this block's results are stored: the wait
            // for its loads then does not wait for those stores as well
            if (hi > RB) store_block(hi - RB, buf0 + (uint32_t)((blk + 1) & 1) * (uint32_t)(RB * 64));
            // buffer row of `newer`: 127 - 16 sb2 - 2 q; the block's rows start at buffer row RB - rows,
            // which is row hi - rows + 1 of the chunk, i.e. time step hi - rows
            const int p_new = 127 - 16 * sb2 - 2 * q;
            const int t_new = hi - rows + (p_new - (RB - rows));
            if (p_new >= RB - rows) {
                st_out[t_new] = (int32_t)(newer & 1023u);
                mv_out[t_new] = (t_new == 0 || !(newer >> 15)) ? (uint8_t)1 : (uint8_t)0;
            }
            if (p_new - 1 >= RB - rows) {
                st_out[t_new - 1] = (int32_t)(older & 1023u);
                mv_out[t_new - 1] = (t_new - 1 == 0 || !(older >> 15)) ? (uint8_t)1 : (uint8_t)0;
            }
        }
    }
}

template <int S, int COLS>
int launch_beam(const void *scores, const float *bwd, ofk_beam_slot_t *beam, int32_t *states,
                uint8_t *moves, int T, int N, float log_cut, float stay, int flags, const double *lse_table,
                hipStream_t st) {
    // 256 compute units: up to 512 chunks fit two to a unit; larger batches go four to a group
    // where the LDS of four chunks fits (64 and 256 states)
    if constexpr (S <= 256) {
        if (N > OFK_SPARSE_SEARCH_MAX_CHUNKS) {
            hipLaunchKernelGGL((beam_kernel<S, 4, COLS>), dim3((N + 3) / 4), dim3(512), 0, st,
                               static_cast<const _Float16 *>(scores), bwd, beam, states, moves, T, N, log_cut,
                               stay, flags, lse_table);
            return (int)hipGetLastError();
        }
    }
    hipLaunchKernelGGL((beam_kernel<S, 2, COLS>), dim3((N + 1) / 2), dim3(256), 0, st,
                           static_cast<const _Float16 *>(scores), bwd, beam, states, moves, T, N, log_cut, stay,
                           flags, lse_table);
    return (int)hipGetLastError();
}

int dispatch_beam(const void *scores, const float *bwd, ofk_beam_slot_t *beam, int32_t *states, uint8_t *moves,
                  int T, int N, int state_len, int columns, float log_cut, float stay, int flags,
                  const double *lse_table, hipStream_t st) {
    switch (state_len * 8 + columns) {
        case 3 * 8 + 4: return launch_beam<64, 4>(scores, bwd, beam, states, moves, T, N, log_cut, stay, flags, lse_table, st);
        case 4 * 8 + 4: return launch_beam<256, 4>(scores, bwd, beam, states, moves, T, N, log_cut, stay, flags, lse_table, st);
        case 5 * 8 + 4: return launch_beam<1024, 4>(scores, bwd, beam, states, moves, T, N, log_cut, stay, flags, lse_table, st);
        case 3 * 8 + 5: return launch_beam<64, 5>(scores, bwd, beam, states, moves, T, N, log_cut, stay, flags, lse_table, st);
        case 4 * 8 + 5: return launch_beam<256, 5>(scores, bwd, beam, states, moves, T, N, log_cut, stay, flags, lse_table, st);
        case 5 * 8 + 5: return launch_beam<1024, 5>(scores, bwd, beam, states, moves, T, N, log_cut, stay, flags, lse_table, st);
        default: return OFK_BAD_ARGS;
    }
}

}  // namespace

// ---------------------------------------------------------------------------------------------
// The same search with its scratch memory (the persisted beam slots the traceback walks, and the
// log-sum-exp table) in a static device array instead of buffers of a gpubuf: for callers that
// must not allocate.  Every GPU the library runs on holds its own copy of the array until the
// process ends; `scratch` below is only the host-side handle of it, the device address comes
// from hipGetSymbolAddress, once per device.
// ---------------------------------------------------------------------------------------------
namespace {

constexpr size_t kStaticTableBytes = 8192;  // 612 doubles, rounded up
static __device__ __align__(256) unsigned char scratch[kStaticTableBytes + OFK_STATIC_SLOT_BYTES];

constexpr int kMaxDevices = 64;
unsigned char *g_scratch_of[kMaxDevices];  // device address of `scratch` per device, once looked up
std::mutex g_scratch_mutex;

}  // namespace

// Set-up of the static scratch array on the current device: looks up the array's device address and
// copies the log-sum-exp table behind it (a blocking copy).  Once per device; later calls return at once.
extern "C" int ofk_beam_search_static_prepare(const double *lse_table_host) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= kMaxDevices) return OFK_BAD_ARGS;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_of[dev]) return 0;
    if (!lse_table_host) return OFK_BAD_ARGS;
    void *p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return (int)e;
    e = hipMemcpy(p, lse_table_host, sizeof(double) * OFK_LSE_DOUBLES, hipMemcpyHostToDevice);
    if (e != hipSuccess) return (int)e;
    g_scratch_of[dev] = static_cast<unsigned char *>(p);
    return 0;
}

// 1 if the current device's array has been set up, 0 if not (or if the device cannot be told)
extern "C" int ofk_beam_search_static_ready(void) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 0;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    return g_scratch_of[dev] ? 1 : 0;
}

extern "C" int ofk_beam_search_static(const void *scores, const float *bwd, int32_t *states, uint8_t *moves, int T,
                                      int N, int state_len, int columns, float log_beam_cut, float stay, int flags,
                                      void *stream) {
    if (!scores || !bwd || !states || !moves || T < 1 || N < 1) return OFK_BAD_ARGS;
    if ((reinterpret_cast<uintptr_t>(scores) | reinterpret_cast<uintptr_t>(bwd)) & 15u) return OFK_BAD_ARGS;
    if ((size_t)N * (size_t)(T + 1) * kW * sizeof(ofk_beam_slot_t) > (size_t)OFK_STATIC_SLOT_BYTES) return OFK_TOO_LARGE;
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= kMaxDevices) return OFK_BAD_ARGS;
    unsigned char *base;
    {
        std::lock_guard<std::mutex> lock(g_scratch_mutex);
        base = g_scratch_of[dev];
    }
    if (!base) return OFK_NOT_PREPARED;
    // nothing in the array has to start at zero: the search writes every slot the traceback reads
    ofk_beam_slot_t *beam = reinterpret_cast<ofk_beam_slot_t *>(base + kStaticTableBytes);
    const double *lse_table = reinterpret_cast<const double *>(base);
    hipStream_t st = static_cast<hipStream_t>(stream);
    return dispatch_beam(scores, bwd, beam, states, moves, T, N, state_len, columns, log_beam_cut, stay, flags,
                         lse_table, st);
}

extern "C" int ofk_beam_search(const void *scores, const float *bwd, ofk_beam_slot_t *beam, int32_t *states,
                               uint8_t *moves, int T, int N, int state_len, int columns, float log_beam_cut,
                               float stay, const double *lse_table, int flags, void *stream) {
    if (!scores || !bwd || !beam || !states || !moves || !lse_table || T < 1 || N < 1) return OFK_BAD_ARGS;
    if ((reinterpret_cast<uintptr_t>(scores) | reinterpret_cast<uintptr_t>(bwd) | reinterpret_cast<uintptr_t>(beam)) & 15u)
        return OFK_BAD_ARGS;
    hipStream_t st = static_cast<hipStream_t>(stream);
    return dispatch_beam(scores, bwd, beam, states, moves, T, N, state_len, columns, log_beam_cut, stay, flags,
                         lse_table, st);
}
