// Backward and forward log-space scans over the 4^state_len CRF states, gfx950.
//
// The k-mer transition graph has a quad structure: the four states {4q+j} share
// the four predecessors {q + b*S/4} and the 16 contiguous scores [16q, 16q+16)
// (element 4j+b is the transition pred b -> state 4q+j).  A lane owns SPL = 4, 2 or 1
// states of one quad:
//   forward : owns SPL consecutive states of the contiguous quad {4q+j}, needs the
//             strided quad of the previous vector (4 LDS reads); its own values
//             stay in registers;
//   backward: owns SPL consecutive members of the strided quad {r + c*S/4}, needs
//             the contiguous quad {4r+b} of the next vector (one 128-bit LDS read).
// Per time step a lane reads its 8*SPL bytes of fp16 scores (a wave reads whole
// rows, every cache line fully used), the state vector is exchanged through LDS
// and, when a chunk fits one wavefront, no block barrier is needed.  SPL is chosen
// at launch so that the batch fills the 1024 SIMDs of the device: few chunks are
// spread over more lanes.  Score rows (and bwd rows in the forward sweep) for the
// next DEPTH time steps are kept in flight in registers.
//
// Arithmetic follows the CPU path (reference src/decode_cpu.c:13-147): fp32
// sums of state value and score, max, exp of the fp32 differences, running sum
// in transition order, max + log(sum).  Three variants of that last step exist:
//   precise : exp and log in double, the running sum rounded to fp32 after every
//             term and one rounding of max + log(sum), i.e. the CPU path's own
//             sequence of roundings (fp64 FMA issues at the fp32 rate on gfx950);
//   fast    : v_exp_f32 / v_log_f32, within an ulp or two of the precise result;
//   two-tier: the fast value wherever it provably rounds like the precise one (its
//             distance to a rounding boundary exceeds a bound on its error), the
//             precise arithmetic for the remaining lanes.  Same bits as precise.
// State values reach several thousand, where one fp32 ulp is already 5e-4, and
// the posterior is exp(fwd + bwd - const): a last-bit difference in a scan shows
// up as a 5e-4 relative difference of a posterior.  Two-tier is the default for
// that reason; fast exists for measurements.
//
// Kernels: bwd_scan_kernel and fwd_post_kernel are the two sweeps one after the other;
// scan_post_kernel runs both sweeps of a chunk in one workgroup, from both ends of the
// chunk towards the middle and on to the other end, and is what a decode uses.
#include <hip/hip_runtime.h>

#include <type_traits>

#include "dmath.h"
#include "kernels.h"

namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));

// fp16 scores per state and time step: the four transitions, or five with an unused blank first.
// The file is compiled once for each layout.
#ifndef OFK_COLS
#define OFK_COLS 4
#endif
constexpr int kCols = OFK_COLS;
constexpr int kLead = kCols - 4;
static_assert(kCols == 4 || kCols == 5, "scores have four or five columns");

constexpr float kLog2e = 1.44269504088896340736f;
constexpr float kLn2 = 0.69314718055994530942f;

template <int CTRL>
__device__ __forceinline__ float dpp(float x) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xF, 0xF, true));
}
__device__ __forceinline__ float lane_value(float x, int lane) {
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(x), lane));
}

// reductions over the lanes of one chunk inside a wave: LANES is 16 (one DPP row),
// 32 or 64 (whole wave).  Every lane of the group ends with the same bits.
template <int LANES>
__device__ __forceinline__ float group_sum(float x) {
    x += dpp<0x128>(x);  // row_ror:8
    x += dpp<0x124>(x);  // row_ror:4
    x += dpp<0x122>(x);  // row_ror:2
    x += dpp<0x121>(x);  // row_ror:1
    if constexpr (LANES >= 64) {
        // row sums travel across the rows: lane 15 of a row into the next row (rows 1 and 3), then
        // lane 31 into rows 2 and 3; lane 63 holds the total
        x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x142 /* row_bcast:15 */, 0xA, 0xF, false));
        x += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x143 /* row_bcast:31 */, 0xC, 0xF, false));
        x = lane_value(x, 63);
    } else if constexpr (LANES == 32) {
        const float lo = lane_value(x, 0) + lane_value(x, 16), hi = lane_value(x, 32) + lane_value(x, 48);
        x = (threadIdx.x & 32) ? hi : lo;
    }
    return x;
}
template <int LANES>
__device__ __forceinline__ float group_max(float x) {
    x = fmaxf(x, dpp<0x128>(x));
    x = fmaxf(x, dpp<0x124>(x));
    x = fmaxf(x, dpp<0x122>(x));
    x = fmaxf(x, dpp<0x121>(x));
    if constexpr (LANES >= 64) {
        x = fmaxf(fmaxf(lane_value(x, 0), lane_value(x, 16)), fmaxf(lane_value(x, 32), lane_value(x, 48)));
    } else if constexpr (LANES == 32) {
        const float lo = fmaxf(lane_value(x, 0), lane_value(x, 16)), hi = fmaxf(lane_value(x, 32), lane_value(x, 48));
        x = (threadIdx.x & 32) ? hi : lo;
    }
    return x;
}

template <bool MULTIWAVE>
__device__ __forceinline__ void chunk_sync() {
    if constexpr (MULTIWAVE) {
        // Only LDS traffic has to be ordered across the barrier.  __syncthreads() would also
        // wait for every global load and store in flight, i.e. drain the prefetch ring at
        // every time step.
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
    } else {
        // one wavefront per chunk: LDS operations of a wave complete in order, only the
        // compiler has to be kept from moving the reads above the writes
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
}

// What the CPU-faithful logarithm reads: its table in LDS and its series coefficients.  The
// coefficients travel as a kernel argument, which puts them into scalar registers for the whole
// kernel (as literals the compiler copies them into vector registers at every use).
struct LogSeries {
    double c[6];
    double e[OFA_EXP_COEF_COUNT];  // exponential: polynomial, rounding shift, log2(e), -ln 2
};
struct LogArgs {
    const ofa::LogCell *cells;
    const double *series;
    const double *expc;
    float *lanes;  // 64 floats of LDS owned by the calling wave (two-tier updates only)
    int hurry = 3;  // the wave's priority during a trip through the second tier
};

// Two-tier update, second tier.  `value` is the estimate of a lane's update, `unsettled` says
// that it may differ from the CPU path's result.  A wave usually has none, one or two such
// lanes, and evaluating the CPU roundings under their execution mask would cost the whole wave
// the five double exponentials, the running sum and the logarithm one after another.  Instead
// the unsettled lanes hand their inputs (d_0..d_4 = v_i - m, and m) to groups of eight lanes
// through LDS: lane 8q+j of group q computes the double exponential of d_j of the q-th unsettled
// lane, the fp32 running sum travels from lane to lane by DPP row shifts (so lane 8q+4 ends with
// the CPU path's sum), that lane takes the logarithm, adds m in double and rounds once, and the
// result returns to its owner through a lane permute.  More than eight unsettled lanes take
// further trips (only the first few dozen time steps have that many: values are small there and
// an ulp is tiny; the kernels run those steps with the double arithmetic throughout).
__device__ __forceinline__ float resolve_unsettled(float value, float sum, bool unsettled, float v0, float v1, float v2,
                                                   float v3, float v4, float m, const LogArgs &logtab) {
    uint64_t mask = __builtin_amdgcn_ballot_w64(unsettled);
    if (mask == 0) return value;
    // the chunk's other waves wait at the barrier for this one
    if (logtab.hurry == 3) __builtin_amdgcn_s_setprio(3);
    else if (logtab.hurry == 2) __builtin_amdgcn_s_setprio(2);
    else if (logtab.hurry == 1) __builtin_amdgcn_s_setprio(1);
    const int lane = threadIdx.x & 63;
    int rank = __builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0));
    if (!unsettled) rank = -1;
    do {  // eight unsettled lanes per trip
        if ((unsigned)rank < 8u) {
            float *slot = logtab.lanes + 8 * rank;
            *reinterpret_cast<float4 *>(slot) = make_float4(v0 - m, v1 - m, v2 - m, v3 - m);
            *reinterpret_cast<float4 *>(slot + 4) = make_float4(v4 - m, m, sum, 0.f);
        }
        const float x = logtab.lanes[lane];  // LDS operations of one wave complete in order
        // lane 8q+4 will take the logarithm: its table cell is fetched now, chosen with the estimate
        // of the sum (two lanes up), and arrives while the exponentials are evaluated
        const float near = dpp<0x102>(x);  // row_shl:2
        const ofa::LogCell cell = ofa::log_cell_near(near, logtab.cells);
        const double e = ofa::exp_ldexp((double)x, logtab.expc);
        float s = (float)e;
#pragma unroll
        for (int k = 0; k < 4; ++k) s = (float)((double)dpp<0x111>(s) + e);  // row_shr:1: the sum so far, from the lane below
        const float m_of_group = dpp<0x101>(x);  // row_shl:1: lane 8q+4 reads m from lane 8q+5
        float r = (float)((double)m_of_group + ofa::log_1to5_with_cell(s, near, cell, logtab.series));
        r = s == 1.0f ? m_of_group : r;  // ln 1 = 0 exactly, as on the CPU path
        const float mine = __int_as_float(__builtin_amdgcn_ds_bpermute((8 * (rank & 7) + 4) << 2, __float_as_int(r)));
        if ((unsigned)rank < 8u) value = mine;
        rank -= 8;
        mask = __builtin_amdgcn_ballot_w64(rank >= 0);
    } while (mask != 0);
    if (logtab.hurry) __builtin_amdgcn_s_setprio(0);
    return value;
}

// maximum of three in one instruction (the operands are never NaN here; fmaxf would first quiet
// each operand that comes out of inline assembly with an extra instruction)
__device__ __forceinline__ float max3(float a, float b, float c) {
    float r;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}

// max + log(sum_i exp(v_i - max)), sum taken in the order v0..v4
template <int MODE>
__device__ __forceinline__ float lse5(float v0, float v1, float v2, float v3, float v4, const LogArgs &logtab) {
    const float m = max3(max3(v0, v1, v2), v3, v4);
    if constexpr (MODE == OFK_SCAN_PRECISE) {
        return ofa::lse5_cpu_rounding_tab(v0, v1, v2, v3, v4, m, logtab.cells, logtab.series, logtab.expc);
    } else if constexpr (MODE == OFK_SCAN_TWO_TIER) {
        const ofa::Lse5Estimate e = ofa::lse5_estimate(v0, v1, v2, v3, v4, m);
        return resolve_unsettled(e.value, e.sum, !e.settled, v0, v1, v2, v3, v4, m, logtab);
    } else {
        float s = __builtin_amdgcn_exp2f((v0 - m) * kLog2e);
        s += __builtin_amdgcn_exp2f((v1 - m) * kLog2e);
        s += __builtin_amdgcn_exp2f((v2 - m) * kLog2e);
        s += __builtin_amdgcn_exp2f((v3 - m) * kLog2e);
        s += __builtin_amdgcn_exp2f((v4 - m) * kLog2e);
        return __builtin_fmaf(__builtin_amdgcn_logf(s), kLn2, m);
    }
}

template <int S, int SPL>
struct Shape {
    static constexpr int kLanes = S / SPL;                            // lanes per chunk
    // Workgroups are four wavefronts wherever a chunk needs fewer: the four waves of a
    // group land on the four SIMDs of a compute unit, while smaller groups were seen
    // to pile up on two of them.  Chunks sharing a group stay independent.
    static constexpr int kChunks = kLanes >= 256 ? 1 : 256 / kLanes;  // chunks per workgroup
    static constexpr int kThreads = kLanes >= 256 ? kLanes : 256;
    static constexpr bool kMultiWave = kLanes > 64;                   // a chunk spans several waves
    static constexpr int kGroup = kLanes >= 64 ? 64 : kLanes;         // chunk lanes inside one wave
    static constexpr int kChunkWaves = kLanes > 64 ? kLanes / 64 : 1;
    static constexpr int kQuarter = S / 4;
};

// The backward sweep keeps its state vector in LDS with the four quarters {c * S/4 ..} spaced
// S/4 + kPad floats apart: a lane stores r + c * S/4, and with S/4 a multiple of the 64 banks
// the lanes of a wave that differ only in c would all hit one bank.  16 floats of padding
// spread them over all banks; reads of the contiguous quad {4r + b} stay 16-byte aligned.
template <int S>
struct BwdVec {
    static constexpr int kQ = S / 4;
    static constexpr int kPad = kQ % 64 == 0 ? 16 : 0;
    static constexpr int kLen = S + 4 * kPad;
    static __device__ __forceinline__ int at(int r, int c) { return r + c * (kQ + kPad); }  // state r + c * S/4, r < S/4
    static __device__ __forceinline__ int of(int s) { return s + kPad * (s / kQ); }         // any state s
};

// x + (float)h for the fp16 value h in the low (HI = 0) or high half of a 32-bit register, in one
// instruction: v_fma_mix_f32 converts the half operand on the fly, the product with 1.0 is
// exact, so the result is the correctly rounded fp32 sum, bit for bit what v_cvt_f32_f16
// followed by v_add_f32 gives (checked for every fp16 bit pattern, subnormals included).
template <int HI>
__device__ __forceinline__ float add_half(uint32_t word, float x) {
    float r;
    if constexpr (HI)
        asm("v_fma_mix_f32 %0, %1, 1.0, %2 op_sel:[1,0,0] op_sel_hi:[1,0,0]" : "=v"(r) : "v"(word), "v"(x));
    else
        asm("v_fma_mix_f32 %0, %1, 1.0, %2 op_sel_hi:[1,0,0]" : "=v"(r) : "v"(word), "v"(x));
    return r;
}

// The scores one lane needs for one time step, as loaded: fp16 pairs in 32-bit words.
// A state's scores are kCols consecutive fp16 values: the four transitions, after kLead
// values that the decoder never reads (the blank column of five-column scores).  With
// four columns a lane's window is contiguous and is fetched with vector loads; with five
// it is fetched straight from the caller's layout, 32 bits at a time where two wanted values
// are neighbours (from addresses that are only 2-byte aligned, which global loads accept), two
// bytes at a time elsewhere.
__device__ __forceinline__ uint32_t half_at(const _Float16 *p) { return *reinterpret_cast<const uint16_t *>(p); }
__device__ __forceinline__ uint32_t half_pair_at(const _Float16 *p) {
    if constexpr (kCols == 4) {
        return *reinterpret_cast<const uint32_t *>(p);
    } else {  // one 32-bit load from an address that is only 2-byte aligned
        uint32_t w;
        __builtin_memcpy(&w, p, 4);
        return w;
    }
}

// Backward: transition b of own state i is element kCols * b + i of the lane's window
// (word (4b + i) / 2 of w once packed).
template <int SPL>
struct BwdRow;
template <>
struct BwdRow<4> {
    uint32_t w[8];
    __device__ __forceinline__ void load(const _Float16 *p) {
        if constexpr (kCols == 4) {
            const uint4 x = reinterpret_cast<const uint4 *>(p)[0], y = reinterpret_cast<const uint4 *>(p)[1];
            w[0] = x.x; w[1] = x.y; w[2] = x.z; w[3] = x.w;
            w[4] = y.x; w[5] = y.y; w[6] = y.z; w[7] = y.w;
        } else {
#pragma unroll
            for (int b = 0; b < 4; ++b) {
                w[2 * b] = half_pair_at(p + kCols * b);
                w[2 * b + 1] = half_pair_at(p + kCols * b + 2);
            }
        }
    }
    template <int B, int I>
    __device__ __forceinline__ float add(float x) const {
        constexpr int e = 4 * B + I;
        return add_half<e % 2>(w[e / 2], x);
    }
};
template <>
struct BwdRow<2> {
    uint32_t v[4];
    __device__ __forceinline__ void load(const _Float16 *p) {
#pragma unroll
        for (int b = 0; b < 4; ++b) v[b] = half_pair_at(p + kCols * b);
    }
    template <int B, int I>
    __device__ __forceinline__ float add(float x) const { return add_half<I>(v[B], x); }
};
template <>
struct BwdRow<1> {
    uint32_t v[4];  // one fp16 value each, in the low half
    __device__ __forceinline__ void load(const _Float16 *p) {
#pragma unroll
        for (int b = 0; b < 4; ++b) v[b] = half_at(p + kCols * b);
    }
    template <int B, int I>
    __device__ __forceinline__ float add(float x) const { return add_half<0>(v[B], x); }
};

// Forward: transition b into own state i is element kCols * i + b of the lane's window
// (word (4i + b) / 2 of w once packed).
template <int SPL>
struct FwdRow {
    uint32_t w[2 * SPL];
    __device__ __forceinline__ void load(const _Float16 *p) {
        if constexpr (kCols == 4 && SPL == 4) {
            const uint4 x = reinterpret_cast<const uint4 *>(p)[0], y = reinterpret_cast<const uint4 *>(p)[1];
            w[0] = x.x; w[1] = x.y; w[2] = x.z; w[3] = x.w;
            w[4] = y.x; w[5] = y.y; w[6] = y.z; w[7] = y.w;
        } else if constexpr (kCols == 4 && SPL == 2) {
            const uint4 x = *reinterpret_cast<const uint4 *>(p);
            w[0] = x.x; w[1] = x.y; w[2] = x.z; w[3] = x.w;
        } else if constexpr (kCols == 4) {
            const uint2 x = *reinterpret_cast<const uint2 *>(p);
            w[0] = x.x; w[1] = x.y;
        } else {
#pragma unroll
            for (int i = 0; i < SPL; ++i) {
                w[2 * i] = half_pair_at(p + kCols * i);
                w[2 * i + 1] = half_pair_at(p + kCols * i + 2);
            }
        }
    }
    template <int I, int B>
    __device__ __forceinline__ float add(float x) const {
        constexpr int e = 4 * I + B;
        return add_half<e % 2>(w[e / 2], x);
    }
};

// SPL consecutive floats in global or shared memory
template <int SPL>
struct FloatRun {
    float v[SPL];
    __device__ __forceinline__ void load(const float *p) {
        if constexpr (SPL == 4) {
            const float4 x = *reinterpret_cast<const float4 *>(p);
            v[0] = x.x; v[1] = x.y; v[2] = x.z; v[3] = x.w;
        } else if constexpr (SPL == 2) {
            const float2 x = *reinterpret_cast<const float2 *>(p);
            v[0] = x.x; v[1] = x.y;
        } else {
            v[0] = *p;
        }
    }
    __device__ __forceinline__ void store(float *p) const {
        if constexpr (SPL == 4) *reinterpret_cast<float4 *>(p) = make_float4(v[0], v[1], v[2], v[3]);
        else if constexpr (SPL == 2) *reinterpret_cast<float2 *>(p) = make_float2(v[0], v[1]);
        else *p = v[0];
    }
};

template <int I, int SPL, int MODE>
__device__ __forceinline__ void bwd_update(float (&a)[SPL], const float4 &nx, const BwdRow<SPL> &row, float stay,
                                           const LogArgs &logtab) {
    if constexpr (I < SPL) {
        a[I] = lse5<MODE>(a[I] + stay, row.template add<0, I>(nx.x), row.template add<1, I>(nx.y),
                          row.template add<2, I>(nx.z), row.template add<3, I>(nx.w), logtab);
        bwd_update<I + 1, SPL, MODE>(a, nx, row, stay, logtab);
    }
}

template <int I, int SPL, int MODE>
__device__ __forceinline__ void fwd_update(float (&f)[SPL], float p0, float p1, float p2, float p3,
                                           const FwdRow<SPL> &row, float stay, const LogArgs &logtab) {
    if constexpr (I < SPL) {
        f[I] = lse5<MODE>(f[I] + stay, row.template add<I, 0>(p0), row.template add<I, 1>(p1),
                          row.template add<I, 2>(p2), row.template add<I, 3>(p3), logtab);
        fwd_update<I + 1, SPL, MODE>(f, p0, p1, p2, p3, row, stay, logtab);
    }
}

// ---------------------------------------------------------------------------
// backward: bwd[n][t][s] for t = T..0
// ---------------------------------------------------------------------------
template <int S, int SPL, int DEPTH, int MODE>
__global__ __launch_bounds__((Shape<S, SPL>::kThreads)) void bwd_scan_kernel(
    const _Float16 *__restrict__ scores, float *__restrict__ bwd, int T, int N, float stay, LogSeries series) {
    using Sh = Shape<S, SPL>;
    constexpr int L = Sh::kLanes;
    constexpr int Q = Sh::kQuarter;
    constexpr int H = 4 / SPL;  // lanes sharing one quad
    using Vec = BwdVec<S>;
    __shared__ __attribute__((aligned(16))) float vec[Sh::kChunks][2][Vec::kLen];
    __shared__ __attribute__((aligned(16))) ofa::LogCell logcells[32];
    __shared__ __attribute__((aligned(16))) float tier_lanes[MODE == OFK_SCAN_TWO_TIER ? Sh::kThreads : 64];
    const int tid = threadIdx.x;
    const LogArgs logtab{logcells, series.c, series.e, tier_lanes + (MODE == OFK_SCAN_TWO_TIER ? (tid & ~63) : 0)};

    if (MODE != OFK_SCAN_FAST && tid < 32) logcells[tid] = ofa::log_cell(tid);
    const int g = tid / L, l = tid % L;
    const int r = l / H, c0 = (l % H) * SPL;  // own states: r + (c0 + i) * Q
    int n = blockIdx.x * Sh::kChunks + g;
    const bool live = n < N;
    if (!live) n = N - 1;

    const size_t row_stride = (size_t)N * kCols * S;  // fp16 elements between time steps
    const _Float16 *sp = scores + (size_t)n * kCols * S + 4 * kCols * r + kLead + c0;
    float *out = bwd + (size_t)n * (size_t)(T + 1) * S + r + c0 * Q;

    float a[SPL];
#pragma unroll
    for (int i = 0; i < SPL; ++i) a[i] = 0.f;
    if (live) {
#pragma unroll
        for (int i = 0; i < SPL; ++i) out[(size_t)T * S + i * Q] = 0.f;
    }

    BwdRow<SPL> ring[DEPTH];
#pragma unroll
    for (int k = 0; k < DEPTH; ++k) {
        const int t = T - 1 - k;
        if (t >= 0) ring[k].load(sp + (size_t)t * row_stride);
    }

    int buf = 0;
#pragma unroll
    for (int i = 0; i < SPL; ++i) vec[g][0][Vec::at(r, c0 + i)] = 0.f;
    __syncthreads();  // the log table is shared by the whole group

    for (int done = 0; done < T; done += DEPTH) {
#pragma unroll
        for (int k = 0; k < DEPTH; ++k) {
            const int t = T - 1 - done - k;
            if (t >= 0) {
                const BwdRow<SPL> row = ring[k];
                if (t - DEPTH >= 0) ring[k].load(sp + (size_t)(t - DEPTH) * row_stride);
                chunk_sync<Sh::kMultiWave>();
                const float4 nx = *reinterpret_cast<const float4 *>(&vec[g][buf][Vec::of(4 * r)]);
                bwd_update<0, SPL, MODE>(a, nx, row, stay, logtab);
                buf ^= 1;
#pragma unroll
                for (int i = 0; i < SPL; ++i) vec[g][buf][Vec::at(r, c0 + i)] = a[i];
                if (live) {
#pragma unroll
                    for (int i = 0; i < SPL; ++i) out[(size_t)t * S + i * Q] = a[i];
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------
// forward + posterior: post[n][t][s] = softmax_s(fwd[t][s] + bwd[n][t][s]), t = 0..T
// ---------------------------------------------------------------------------
template <int S, int SPL, int DEPTH, int MODE>
__global__ __launch_bounds__((Shape<S, SPL>::kThreads)) void fwd_post_kernel(
    const _Float16 *__restrict__ scores, const float *__restrict__ bwd, float *__restrict__ post, int T,
    int N, float stay, LogSeries series) {
    using Sh = Shape<S, SPL>;
    constexpr int L = Sh::kLanes;
    constexpr int Q = Sh::kQuarter;
    __shared__ __attribute__((aligned(16))) float vec[Sh::kChunks][2][S];
    __shared__ float part[2][Sh::kChunks][Sh::kChunkWaves];
    __shared__ __attribute__((aligned(16))) ofa::LogCell logcells[32];
    __shared__ __attribute__((aligned(16))) float tier_lanes[MODE == OFK_SCAN_TWO_TIER ? Sh::kThreads : 64];
    const int tid = threadIdx.x;
    // this sweep runs beside the beam search, whose waves run at priority 3: trips through the second tier
    // at 1 leave that search alone (2048 chunks of 64 states: search 2.50 ms against 2.59 with 3 here)
    const LogArgs logtab{logcells, series.c, series.e, tier_lanes + (MODE == OFK_SCAN_TWO_TIER ? (tid & ~63) : 0), 1};

    if (MODE != OFK_SCAN_FAST && tid < 32) logcells[tid] = ofa::log_cell(tid);
    const int g = tid / L, l = tid % L;
    const int s0 = SPL * l, q = s0 >> 2;  // own states s0 .. s0+SPL-1, all in quad q
    const int wave = l / 64;  // wave within the chunk
    int n = blockIdx.x * Sh::kChunks + g;
    const bool live = n < N;
    if (!live) n = N - 1;

    const size_t row_stride = (size_t)N * kCols * S;
    const _Float16 *sp = scores + (size_t)n * kCols * S + kCols * s0 + kLead;
    const float *bp = bwd + (size_t)n * (size_t)(T + 1) * S + s0;
    float *pp = post + (size_t)n * (size_t)(T + 1) * S + s0;

    FwdRow<SPL> ring[DEPTH];
    FloatRun<SPL> bring[DEPTH];
#pragma unroll
    for (int k = 0; k < DEPTH; ++k) {
        if (k < T) ring[k].load(sp + (size_t)k * row_stride);
        if (k <= T) bring[k].load(bp + (size_t)k * S);
    }

    // Shift of the softmax exponent.  sum_s exp(fwd+bwd) is the same partition function at
    // every time step, and at t = 0 it lies within log(S) of max_s bwd[0][s]; that maximum,
    // lowered by 10 so that tiny posteriors stay normal numbers until the final product,
    // replaces the per-step maximum (the quotient does not depend on the shift).
    float shift;
    {
        FloatRun<SPL> b0;
        b0.load(bp);
        float m = b0.v[0];
#pragma unroll
        for (int i = 1; i < SPL; ++i) m = fmaxf(m, b0.v[i]);
        m = group_max<Sh::kGroup>(m);
        if constexpr (Sh::kMultiWave) {
            if ((tid & 63) == 0) part[0][g][wave] = m;
            chunk_sync<true>();
            m = part[0][g][0];
#pragma unroll
            for (int w = 1; w < Sh::kChunkWaves; ++w) m = fmaxf(m, part[0][g][w]);
            chunk_sync<true>();
        }
        shift = m - 10.0f;
    }

    float f[SPL];
#pragma unroll
    for (int i = 0; i < SPL; ++i) f[i] = 0.f;
    int buf = 0;
    __syncthreads();  // the log table is shared by the whole group

    for (int done = 0; done <= T; done += DEPTH) {
#pragma unroll
        for (int k = 0; k < DEPTH; ++k) {
            const int t = done + k;
            if (t <= T) {
                const FwdRow<SPL> row = ring[k];
                const FloatRun<SPL> bw = bring[k];
                if (t + DEPTH < T) ring[k].load(sp + (size_t)(t + DEPTH) * row_stride);
                if (t + DEPTH <= T) bring[k].load(bp + (size_t)(t + DEPTH) * S);

                // posterior of time step t
                FloatRun<SPL> e;
                float total = 0.f;
#pragma unroll
                for (int i = 0; i < SPL; ++i) {
                    e.v[i] = __builtin_amdgcn_exp2f(((f[i] + bw.v[i]) - shift) * kLog2e);
                    total += e.v[i];
                }
                total = group_sum<Sh::kGroup>(total);

                FloatRun<SPL> mine;
#pragma unroll
                for (int i = 0; i < SPL; ++i) mine.v[i] = f[i];
                mine.store(&vec[g][buf][s0]);
                if constexpr (Sh::kMultiWave) {
                    if ((tid & 63) == 0) part[buf][g][wave] = total;
                }
                chunk_sync<Sh::kMultiWave>();
                if constexpr (Sh::kMultiWave) {
                    total = part[buf][g][0];
#pragma unroll
                    for (int w = 1; w < Sh::kChunkWaves; ++w) total += part[buf][g][w];
                }
                const float inv = __builtin_amdgcn_rcpf(total);
#pragma unroll
                for (int i = 0; i < SPL; ++i) e.v[i] *= inv;
                if (live) e.store(pp + (size_t)t * S);

                if (t < T) {
                    const float p0 = vec[g][buf][q];
                    const float p1 = vec[g][buf][q + Q];
                    const float p2 = vec[g][buf][q + 2 * Q];
                    const float p3 = vec[g][buf][q + 3 * Q];
                    fwd_update<0, SPL, MODE>(f, p0, p1, p2, p3, row, stay, logtab);
                    buf ^= 1;
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------
// forward + posterior with the two jobs on different waves.
//
// fwd_post_kernel's lanes take the posterior of a row between two steps of the recursion: an
// exponential, a sum over the wave, a partial sum through LDS, a reciprocal and a store join the
// chain of dependent operations of every time step, which is what this sweep's duration is made
// of (it runs beside the beam search with two waves per SIMD; 512 chunks of 256 states: 1.41 ms
// against 0.95 ms for the backward sweep, which has no such work).  Here a chunk has twice the
// lanes: one half runs the recursion alone, the other half reads every row the first half
// publishes in LDS for its own exchange anyway, and forms that row's posterior one step behind.
// Every wave takes one block barrier per time step (plus one at the end and two for the shift).
// Same arithmetic, same results.  (Letting the second half also sum the finished row over every
// state's neighbours for the quality stage was measured and dropped: the extra LDS traffic slowed
// the recursion by more, 0.18 ms, than the sums save that stage, 0.09 ms.)
// ---------------------------------------------------------------------------
template <int S, int SPL, int DEPTH>
__global__ __launch_bounds__((2 * (S / SPL))) void fwd_post_roles_kernel(
    const _Float16 *__restrict__ scores, const float *__restrict__ bwd, float *__restrict__ post, int T,
    int N, float stay, LogSeries series) {
    constexpr int L = S / SPL;  // lanes of either job
    constexpr int Q = S / 4;
    constexpr int RW = L / 64;  // waves of either job
    static_assert(L % 64 == 0 && RW > 1, "either job owns several whole waves");
    __shared__ __attribute__((aligned(16))) float vec[2][S];
    __shared__ float part[2][RW];
    __shared__ __attribute__((aligned(16))) ofa::LogCell logcells[32];
    __shared__ __attribute__((aligned(16))) float tier_lanes[L];
    const int tid = threadIdx.x;
    const int posterior = __builtin_amdgcn_readfirstlane(tid / L);
    const int l = tid % L, lane = tid & 63, wave = l / 64;
    // this kernel runs beside the beam search, whose waves run at priority 3: trips through the second
    // tier at 1 leave that search alone (1.17 ms against 1.22 with 3 here) and cost this sweep nothing
    const LogArgs logtab{logcells, series.c, series.e, tier_lanes + (l & ~63), 1};
    if (tid < 32) logcells[tid] = ofa::log_cell(tid);
    const int s0 = SPL * l, q = s0 >> 2;  // own states s0 .. s0+SPL-1, all in quad q
    const int n = blockIdx.x;            // one chunk per workgroup
    const size_t row_stride = (size_t)N * kCols * S;
    auto barrier = [] { chunk_sync<true>(); };

    if (!posterior) {
        const _Float16 *sp = scores + (size_t)n * kCols * S + kCols * s0 + kLead;
        FwdRow<SPL> ring[DEPTH];
#pragma unroll
        for (int k = 0; k < DEPTH; ++k) {
            if (k < T) ring[k].load(sp + (size_t)k * row_stride);
        }
        float f[SPL];
#pragma unroll
        for (int i = 0; i < SPL; ++i) f[i] = 0.f;
        int buf = 0;
        barrier();  // the other half exchanges the maxima behind the shift
        barrier();
        __syncthreads();  // the log table
        for (int done = 0; done <= T; done += DEPTH) {
#pragma unroll
            for (int k = 0; k < DEPTH; ++k) {
                const int t = done + k;
                if (t <= T) {
                    const FwdRow<SPL> row = ring[k];
                    if (t + DEPTH < T) ring[k].load(sp + (size_t)(t + DEPTH) * row_stride);
                    FloatRun<SPL> mine;
#pragma unroll
                    for (int i = 0; i < SPL; ++i) mine.v[i] = f[i];
                    mine.store(&vec[buf][s0]);  // row t
                    barrier();
                    if (t < T) {
                        const float p0 = vec[buf][q], p1 = vec[buf][q + Q];
                        const float p2 = vec[buf][q + 2 * Q], p3 = vec[buf][q + 3 * Q];
                        fwd_update<0, SPL, OFK_SCAN_TWO_TIER>(f, p0, p1, p2, p3, row, stay, logtab);
                        buf ^= 1;
                    }
                }
            }
        }
        barrier();  // the other half finishes row T
    } else {
        const float *bp = bwd + (size_t)n * (size_t)(T + 1) * S + s0;
        float *pp = post + (size_t)n * (size_t)(T + 1) * S + s0;
        FloatRun<SPL> bring[DEPTH];
#pragma unroll
        for (int k = 0; k < DEPTH; ++k) {
            if (k <= T) bring[k].load(bp + (size_t)k * S);
        }
        // Shift of the softmax exponent, as in fwd_post_kernel: max_s bwd[0][s] - 10.
        float shift;
        {
            float m = bring[0].v[0];
#pragma unroll
            for (int i = 1; i < SPL; ++i) m = fmaxf(m, bring[0].v[i]);
            m = group_max<64>(m);
            if (lane == 0) part[0][wave] = m;
            barrier();
            m = part[0][0];
#pragma unroll
            for (int w = 1; w < RW; ++w) m = fmaxf(m, part[0][w]);
            barrier();
            shift = m - 10.0f;
        }
        __syncthreads();
        FloatRun<SPL> e;  // terms of the row before, waiting for the sum over the waves
        int buf = 0;
        auto finish_row = [&](int t) {
            float total = part[t & 1][0];
#pragma unroll
            for (int w = 1; w < RW; ++w) total += part[t & 1][w];
            const float inv = __builtin_amdgcn_rcpf(total);
#pragma unroll
            for (int i = 0; i < SPL; ++i) e.v[i] *= inv;
            e.store(pp + (size_t)t * S);
        };
        for (int done = 0; done <= T; done += DEPTH) {
#pragma unroll
            for (int k = 0; k < DEPTH; ++k) {
                const int t = done + k;
                if (t <= T) {
                    const FloatRun<SPL> bw = bring[k];
                    if (t + DEPTH <= T) bring[k].load(bp + (size_t)(t + DEPTH) * S);
                    barrier();  // row t is in vec[buf], the partial sums of row t - 1 in part[(t - 1) & 1]
                    if (t > 0) finish_row(t - 1);
                    FloatRun<SPL> fv;
                    fv.load(&vec[buf][s0]);
                    buf ^= 1;
                    float total = 0.f;
#pragma unroll
                    for (int i = 0; i < SPL; ++i) {
                        e.v[i] = __builtin_amdgcn_exp2f(((fv.v[i] + bw.v[i]) - shift) * kLog2e);
                        total += e.v[i];
                    }
                    total = group_sum<64>(total);
                    if (lane == 0) part[t & 1][wave] = total;
                }
            }
        }
        barrier();
        finish_row(T);
    }
}

// ---------------------------------------------------------------------------
// Both sweeps in one kernel, meeting in the middle.
//
// The forward recursion does not depend on the backward one; only the posterior needs
// both.  A chunk is served by two groups of lanes of one workgroup, one per direction,
// which doubles the wavefronts in flight (the separate sweeps leave the device at one or
// two waves per SIMD at 512 chunks of 256 states, where every wave issues at half the rate
// the SIMD could take).
//   phase 1: the backward lanes run t = T-1 .. H and write bwd[t]; the forward lanes run
//            t = 0 .. H-1 and park fwd[t] in post[t];
//   middle : the partition function max_s(fwd[H][s] + bwd[H][s]) fixes the exponent shift
//            of the softmax (it is the same at every time step);
//   phase 2: the forward lanes run t = H .. T reading bwd[t] (written in phase 1), the
//            backward lanes run t = H-1 .. 0 reading the parked fwd[t]; both write the
//            posterior, the backward lanes over the parked values.
// HBM traffic: every score twice, bwd written once, half of it read once, post written once
// and half of it written and read once more as fwd: (T+1) S 4 bytes above the two separate
// sweeps.  One block barrier per time step serves both directions.
// ---------------------------------------------------------------------------
template <int S, int SPL>
struct FusedShape {
    static constexpr int kLanes = S / SPL;                 // lanes per direction and chunk
    static constexpr int kRoleWaves = kLanes / 64;         // whole waves: a wave has one direction
    static constexpr int kChunkThreads = 2 * kLanes;
    static constexpr int kChunks = kChunkThreads >= 512 ? 1 : 512 / kChunkThreads;
    static constexpr int kThreads = kChunks * kChunkThreads;
    static constexpr int kQuarter = S / 4;
    static_assert(kLanes % 64 == 0, "a direction owns whole wavefronts");
};

template <int N, typename F>
__device__ __forceinline__ void static_for(F &&f) {
    if constexpr (N > 0) {
        static_for<N - 1>(f);
        f(std::integral_constant<int, N - 1>{});
    }
}

// `count` steps, DEPTH of them unrolled per trip: step(k, j, checked) with k = j % DEPTH a
// compile-time index; in unchecked trips j + DEPTH + SLACK < count holds for every step, i.e.
// every prefetch DEPTH steps ahead is in range (of a tensor with SLACK rows fewer than steps).
template <int DEPTH, int SLACK = 0, typename Step>
__device__ __forceinline__ void pipelined(int count, Step &&step) {
    int j0 = 0;
    for (; j0 + 2 * DEPTH + SLACK <= count; j0 += DEPTH)
        static_for<DEPTH>([&](auto k) { step(k, j0 + (int)k, std::false_type{}); });
    for (; j0 < count; j0 += DEPTH)
        static_for<DEPTH>([&](auto k) {
            if (j0 + (int)k < count) step(k, j0 + (int)k, std::true_type{});
        });
}

__device__ __forceinline__ void block_barrier_lds() { chunk_sync<true>(); }

template <int S, int SPL, int DEPTH, int MODE>
__global__ __launch_bounds__((FusedShape<S, SPL>::kThreads), 4) void scan_post_kernel(
    const _Float16 *__restrict__ scores, float *__restrict__ bwd, float *__restrict__ post, int T, int N, float stay,
    LogSeries series) {
    using Sh = FusedShape<S, SPL>;
    constexpr int L = Sh::kLanes;
    constexpr int Q = Sh::kQuarter;
    constexpr int RW = Sh::kRoleWaves;
    constexpr int H4 = 4 / SPL;  // backward lanes sharing one quad
    constexpr int kWarmup = 32;  // time steps of either sweep evaluated in double before the two tiers take over
    // Per time step the lanes of one direction exchange their state vector (and the partial sums of
    // the posterior's denominator) through LDS.  With several waves per direction that takes a
    // workgroup barrier, which both directions (and every chunk of the group) then share; when a
    // direction is a single wave (64 states), a time step only needs the wave's own LDS operations
    // kept in order, and the waves of a group run their steps without waiting for one another.  The
    // two directions of a chunk meet only in the middle, at block barriers that every wave reaches.
    auto step_sync = [] { chunk_sync<(RW > 1)>(); };
    using VecB = BwdVec<S>;
    __shared__ __attribute__((aligned(16))) float vecB[Sh::kChunks][2][VecB::kLen];
    __shared__ __attribute__((aligned(16))) float vecF[Sh::kChunks][2][S];
    __shared__ float part[Sh::kChunks][2][2][RW];  // [chunk][direction][parity][wave]
    __shared__ float shift_of[Sh::kChunks];
    __shared__ __attribute__((aligned(16))) ofa::LogCell logcells[32];
    __shared__ __attribute__((aligned(16))) float tier_lanes[MODE == OFK_SCAN_TWO_TIER ? Sh::kThreads : 64];
    const int tid = threadIdx.x;
    const LogArgs logtab{logcells, series.c, series.e, tier_lanes + (MODE == OFK_SCAN_TWO_TIER ? (tid & ~63) : 0)};

    if (MODE != OFK_SCAN_FAST && tid < 32) logcells[tid] = ofa::log_cell(tid);
    const int g = tid / Sh::kChunkThreads, u = tid % Sh::kChunkThreads;
    const int forward = __builtin_amdgcn_readfirstlane(u / L);
    const int l = u % L, wave = l / 64;
    int n = blockIdx.x * Sh::kChunks + g;
    const bool live = Sh::kChunks == 1 || n < N;
    if (!live) n = N - 1;

    const int H = T / 2;  // forward: rows 0..H-1 in phase 1, H..T in phase 2
    // Addresses are a base that is the same for the whole workgroup (kept in scalar registers and
    // stepped from row to row by scalar additions) plus a 32-bit offset of the lane that never changes.
    const ptrdiff_t row_stride = (ptrdiff_t)N * kCols * S;  // fp16 elements between time steps
    const int first_chunk = blockIdx.x * Sh::kChunks;
    const unsigned g_eff = (unsigned)(n - first_chunk);  // chunk within the group (dead lanes repeat the last chunk)
    const _Float16 *const sc_blk = scores + (size_t)first_chunk * kCols * S;
    const size_t blk_off = (size_t)first_chunk * (size_t)(T + 1) * S;
    float *const bwd_blk = bwd + blk_off;
    float *const post_blk = post + blk_off;
    const unsigned chunk_rows = g_eff * (unsigned)(T + 1) * S;

    if (!forward) {
        // ------------------------------ backward lanes ------------------------------
        const int r = l / H4, c0 = (l % H4) * SPL;  // own states: r + (c0 + i) * Q
        const unsigned sc_lane = g_eff * kCols * S + 4 * kCols * r + kLead + c0;
        const unsigned st_lane = chunk_rows + r + c0 * Q;
        float a[SPL];
#pragma unroll
        for (int i = 0; i < SPL; ++i) {
            a[i] = 0.f;
            vecB[g][0][VecB::at(r, c0 + i)] = 0.f;
            if (live) bwd_blk[(size_t)T * S + st_lane + i * Q] = 0.f;
        }
        int buf = 0;
        BwdRow<SPL> ring[DEPTH];
        __syncthreads();  // log table, initial vectors

        // phase 1: t = T-1 .. H.  Values start at zero, where an ulp is far below the error bound of
        // the estimate: in two-tier mode the first kWarmup steps use the double arithmetic throughout.
        const int cnt1 = T - H;
        auto sweep1 = [&](auto mode, int first, int count) {
            constexpr int M = decltype(mode)::value;
            const _Float16 *pre = sc_blk + (ptrdiff_t)(T - 1 - first) * row_stride;  // next row to fetch
            float *orow = bwd_blk + (ptrdiff_t)(T - 1 - first) * S;
            static_for<DEPTH>([&](auto k) {
                if ((int)k < count) {
                    ring[k].load(pre + sc_lane);
                    pre -= row_stride;
                }
            });
            pipelined<DEPTH>(count, [&](auto k, int j, auto checked) {
                const BwdRow<SPL> row = ring[k];
                if (!checked || j + DEPTH < count) {
                    ring[k].load(pre + sc_lane);
                    pre -= row_stride;
                }
                step_sync();
                const float4 nx = *reinterpret_cast<const float4 *>(&vecB[g][buf][VecB::of(4 * r)]);
                bwd_update<0, SPL, M>(a, nx, row, stay, logtab);
                buf ^= 1;
#pragma unroll
                for (int i = 0; i < SPL; ++i) vecB[g][buf][VecB::at(r, c0 + i)] = a[i];
                if (live) {
#pragma unroll
                    for (int i = 0; i < SPL; ++i) orow[st_lane + i * Q] = a[i];
                }
                orow -= S;
            });
        };
        const int warm = MODE == OFK_SCAN_TWO_TIER ? (cnt1 < kWarmup ? cnt1 : kWarmup) : 0;
        if constexpr (MODE == OFK_SCAN_TWO_TIER) sweep1(std::integral_constant<int, OFK_SCAN_PRECISE>{}, 0, warm);
        sweep1(std::integral_constant<int, MODE>{}, warm, cnt1 - warm);
        // forward lanes may run one step fewer in phase 1: cnt1 - H is 0 or 1; they wait here
        // middle: bwd[H..T] visible to the forward lanes, fwd[0..H-1] to these; the shift
        __syncthreads();
        block_barrier_lds();  // the forward lanes exchange their partial maxima
        block_barrier_lds();  // ... and publish the shift
        const float shift = shift_of[g];

        // phase 2: t = H-1 .. 0, posterior of row t from the parked fwd[t]
        const int cnt2 = H;
        int pb = 0;
        float e_prev[SPL];
        {
            const _Float16 *pre = sc_blk + (ptrdiff_t)(H - 1) * row_stride;
            const float *fpre = post_blk + (ptrdiff_t)(H - 1) * S;  // next parked row to fetch
            float *orow = bwd_blk + (ptrdiff_t)(H - 1) * S;
            float *prow = post_blk + (ptrdiff_t)H * S;  // row of the posterior that is stored next (one step late)
            float fring[DEPTH][SPL];
            static_for<DEPTH>([&](auto k) {
                if ((int)k < cnt2) {
                    ring[k].load(pre + sc_lane);
#pragma unroll
                    for (int i = 0; i < SPL; ++i) fring[k][i] = fpre[st_lane + i * Q];
                    pre -= row_stride;
                    fpre -= S;
                }
            });
            pipelined<DEPTH>(cnt2, [&](auto k, int j, auto checked) {
                const BwdRow<SPL> row = ring[k];
                float fv[SPL];
#pragma unroll
                for (int i = 0; i < SPL; ++i) fv[i] = fring[k][i];
                if (!checked || j + DEPTH < cnt2) {
                    ring[k].load(pre + sc_lane);
#pragma unroll
                    for (int i = 0; i < SPL; ++i) fring[k][i] = fpre[st_lane + i * Q];
                    pre -= row_stride;
                    fpre -= S;
                }
                step_sync();
                if (j > 0) {  // posterior of the previous row: its total is complete now
                    float total = part[g][0][pb ^ 1][0];
#pragma unroll
                    for (int w = 1; w < RW; ++w) total += part[g][0][pb ^ 1][w];
                    const float inv = __builtin_amdgcn_rcpf(total);
                    if (live) {
#pragma unroll
                        for (int i = 0; i < SPL; ++i) prow[st_lane + i * Q] = e_prev[i] * inv;
                    }
                }
                prow -= S;
                const float4 nx = *reinterpret_cast<const float4 *>(&vecB[g][buf][VecB::of(4 * r)]);
                bwd_update<0, SPL, MODE>(a, nx, row, stay, logtab);
                buf ^= 1;
                float total;
#pragma unroll
                for (int i = 0; i < SPL; ++i) {
                    vecB[g][buf][VecB::at(r, c0 + i)] = a[i];
                    e_prev[i] = __builtin_amdgcn_exp2f(((fv[i] + a[i]) - shift) * kLog2e);
                    total = i ? total + e_prev[i] : e_prev[i];
                }
                total = group_sum<64>(total);
                if ((tid & 63) == 0) part[g][0][pb][wave] = total;
                pb ^= 1;
                if (live) {
#pragma unroll
                    for (int i = 0; i < SPL; ++i) orow[st_lane + i * Q] = a[i];
                }
                orow -= S;
            });
        }
        step_sync();
        if (cnt2 > 0) {
            float total = part[g][0][pb ^ 1][0];
#pragma unroll
            for (int w = 1; w < RW; ++w) total += part[g][0][pb ^ 1][w];
            const float inv = __builtin_amdgcn_rcpf(total);
            if (live) {
#pragma unroll
                for (int i = 0; i < SPL; ++i) post_blk[st_lane + i * Q] = e_prev[i] * inv;  // row 0
            }
        }
        // the forward lanes take T - H + 1 barriers in phase 2, these took H + 1
        for (int x = H + 1; x < T - H + 1; ++x) step_sync();
    } else {
        // ------------------------------ forward lanes ------------------------------
        const int s0 = SPL * l, q = s0 >> 2;  // own states s0 .. s0+SPL-1, all in quad q
        const unsigned sc_lane = g_eff * kCols * S + kCols * s0 + kLead;
        const unsigned st_lane = chunk_rows + s0;
        float f[SPL];
#pragma unroll
        for (int i = 0; i < SPL; ++i) {
            f[i] = 0.f;
            vecF[g][0][s0 + i] = 0.f;
        }
        int buf = 0;
        FwdRow<SPL> ring[DEPTH];
        __syncthreads();

        // phase 1: t = 0 .. H-1, fwd[t] parked in post[t]; warm-up as for the backward lanes
        const int cnt1 = H;
        auto sweep1 = [&](auto mode, int first, int count) {
            constexpr int M = decltype(mode)::value;
            const _Float16 *pre = sc_blk + (ptrdiff_t)first * row_stride;
            float *prow = post_blk + (size_t)first * S;
            static_for<DEPTH>([&](auto k) {
                if ((int)k < count) {
                    ring[k].load(pre + sc_lane);
                    pre += row_stride;
                }
            });
            pipelined<DEPTH>(count, [&](auto k, int j, auto checked) {
                const FwdRow<SPL> row = ring[k];
                if (!checked || j + DEPTH < count) {
                    ring[k].load(pre + sc_lane);
                    pre += row_stride;
                }
                if (live) {
                    FloatRun<SPL> mine;
#pragma unroll
                    for (int i = 0; i < SPL; ++i) mine.v[i] = f[i];
                    mine.store(prow + st_lane);
                }
                prow += S;
                step_sync();
                const float p0 = vecF[g][buf][q], p1 = vecF[g][buf][q + Q];
                const float p2 = vecF[g][buf][q + 2 * Q], p3 = vecF[g][buf][q + 3 * Q];
                fwd_update<0, SPL, M>(f, p0, p1, p2, p3, row, stay, logtab);
                buf ^= 1;
                FloatRun<SPL> mine;
#pragma unroll
                for (int i = 0; i < SPL; ++i) mine.v[i] = f[i];
                mine.store(&vecF[g][buf][s0]);
            });
        };
        const int warm = MODE == OFK_SCAN_TWO_TIER ? (cnt1 < kWarmup ? cnt1 : kWarmup) : 0;
        if constexpr (MODE == OFK_SCAN_TWO_TIER) sweep1(std::integral_constant<int, OFK_SCAN_PRECISE>{}, 0, warm);
        sweep1(std::integral_constant<int, MODE>{}, warm, cnt1 - warm);
        for (int x = cnt1; x < T - H; ++x) step_sync();  // the backward lanes' extra step

        // middle: shift = max_s(fwd[H][s] + bwd[H][s]) - 10
        __syncthreads();
        {
            const int bbuf = (T - H) & 1;  // where the backward lanes left bwd[H]
            FloatRun<SPL> bh;
            bh.load(&vecB[g][bbuf][VecB::of(s0)]);
            float m = f[0] + bh.v[0];
#pragma unroll
            for (int i = 1; i < SPL; ++i) m = fmaxf(m, f[i] + bh.v[i]);
            m = group_max<64>(m);
            if ((tid & 63) == 0) part[g][1][0][wave] = m;
            block_barrier_lds();
            m = part[g][1][0][0];
#pragma unroll
            for (int w = 1; w < RW; ++w) m = fmaxf(m, part[g][1][0][w]);
            if (l == 0) shift_of[g] = m - 10.0f;
            block_barrier_lds();
        }
        const float shift = shift_of[g];

        // phase 2: rows t = H .. T
        const int cnt2 = T - H + 1;
        int pb = 1;  // parity 0 of part[][1] was used for the maximum just now
        {
            const _Float16 *pre = sc_blk + (ptrdiff_t)H * row_stride;
            const float *bpre = bwd_blk + (size_t)H * S;
            float *prow = post_blk + (size_t)H * S;
            FloatRun<SPL> bring[DEPTH];
            static_for<DEPTH>([&](auto k) {
                if ((int)k < cnt2 - 1) ring[k].load(pre + sc_lane);
                if ((int)k < cnt2) bring[k].load(bpre + st_lane);
                pre += row_stride;
                bpre += S;
            });
            pipelined<DEPTH, 1>(cnt2, [&](auto k, int j, auto checked) {
                const FwdRow<SPL> row = ring[k];
                const FloatRun<SPL> bw = bring[k];
                if (!checked || j + DEPTH < cnt2 - 1) ring[k].load(pre + sc_lane);
                if (!checked || j + DEPTH < cnt2) bring[k].load(bpre + st_lane);
                pre += row_stride;
                bpre += S;
                FloatRun<SPL> e;
                float total;
#pragma unroll
                for (int i = 0; i < SPL; ++i) {
                    e.v[i] = __builtin_amdgcn_exp2f(((f[i] + bw.v[i]) - shift) * kLog2e);
                    total = i ? total + e.v[i] : e.v[i];
                }
                total = group_sum<64>(total);
                if ((tid & 63) == 0) part[g][1][pb][wave] = total;
                step_sync();
                total = part[g][1][pb][0];
#pragma unroll
                for (int w = 1; w < RW; ++w) total += part[g][1][pb][w];
                pb ^= 1;
                const float inv = __builtin_amdgcn_rcpf(total);
#pragma unroll
                for (int i = 0; i < SPL; ++i) e.v[i] *= inv;
                if (live) e.store(prow + st_lane);
                prow += S;
                if (!checked || j + 1 < cnt2) {
                    const float p0 = vecF[g][buf][q], p1 = vecF[g][buf][q + Q];
                    const float p2 = vecF[g][buf][q + 2 * Q], p3 = vecF[g][buf][q + 3 * Q];
                    fwd_update<0, SPL, MODE>(f, p0, p1, p2, p3, row, stay, logtab);
                    buf ^= 1;
                    FloatRun<SPL> mine;
#pragma unroll
                    for (int i = 0; i < SPL; ++i) mine.v[i] = f[i];
                    mine.store(&vecF[g][buf][s0]);
                }
            });
        }
    }
}

const LogSeries kSeries = {OFA_LOG_SERIES, OFA_EXP_COEFS};

// The always-double and the hardware-only arithmetic exist for tests and measurements: they are
// built with the fewest states per lane only (the entry points below ask for nothing else).
template <int S>
constexpr int kPlainSpl = S >= 1024 ? 2 : 1;

template <int S, int SPL, int DEPTH>
int launch_bwd(int mode, const void *scores, float *bwd, int T, int N, float stay, hipStream_t st) {
    using Sh = Shape<S, SPL>;
    const dim3 grid((N + Sh::kChunks - 1) / Sh::kChunks), block(Sh::kThreads);
    const _Float16 *sc = static_cast<const _Float16 *>(scores);
    switch (mode) {
        case OFK_SCAN_TWO_TIER:
            hipLaunchKernelGGL((bwd_scan_kernel<S, SPL, DEPTH, OFK_SCAN_TWO_TIER>), grid, block, 0, st, sc, bwd, T, N, stay, kSeries);
            break;
        case OFK_SCAN_PRECISE:
            if constexpr (SPL == kPlainSpl<S>)
                hipLaunchKernelGGL((bwd_scan_kernel<S, SPL, DEPTH, OFK_SCAN_PRECISE>), grid, block, 0, st, sc, bwd, T, N, stay, kSeries);
            else
                return OFK_BAD_ARGS;
            break;
        case OFK_SCAN_FAST:
            if constexpr (SPL == kPlainSpl<S>)
                hipLaunchKernelGGL((bwd_scan_kernel<S, SPL, DEPTH, OFK_SCAN_FAST>), grid, block, 0, st, sc, bwd, T, N, stay, kSeries);
            else
                return OFK_BAD_ARGS;
            break;
        default: return OFK_BAD_ARGS;
    }
    return (int)hipGetLastError();
}

template <int S, int SPL, int DEPTH>
int launch_fwd(int mode, const void *scores, const float *bwd, float *post, int T, int N, float stay, hipStream_t st) {
    using Sh = Shape<S, SPL>;
    const dim3 grid((N + Sh::kChunks - 1) / Sh::kChunks), block(Sh::kThreads);
    const _Float16 *sc = static_cast<const _Float16 *>(scores);
    switch (mode) {
        case OFK_SCAN_TWO_TIER:
            // Recursion and posterior on separate waves, one chunk per group of twice the lanes: where a chunk
            // spans several waves, and while that leaves every SIMD at most four of them (measured, 256 states:
            // 512 chunks 1.17 ms against 1.41 ms beside the beam search, 1024 chunks 3.5 against 3.1)
            if constexpr (Sh::kMultiWave && 2 * Sh::kLanes <= 1024) {
                if ((long)N * (2 * Sh::kLanes / 64) <= 4096) {
                    hipLaunchKernelGGL((fwd_post_roles_kernel<S, SPL, DEPTH>), dim3(N), dim3(2 * Sh::kLanes), 0, st, sc, bwd, post,
                                       T, N, stay, kSeries);
                    break;
                }
            }
            hipLaunchKernelGGL((fwd_post_kernel<S, SPL, DEPTH, OFK_SCAN_TWO_TIER>), grid, block, 0, st, sc, bwd, post, T, N, stay, kSeries);
            break;
        case OFK_SCAN_PRECISE:
            if constexpr (SPL == kPlainSpl<S>)
                hipLaunchKernelGGL((fwd_post_kernel<S, SPL, DEPTH, OFK_SCAN_PRECISE>), grid, block, 0, st, sc, bwd, post, T, N, stay, kSeries);
            else
                return OFK_BAD_ARGS;
            break;
        case OFK_SCAN_FAST:
            if constexpr (SPL == kPlainSpl<S>)
                hipLaunchKernelGGL((fwd_post_kernel<S, SPL, DEPTH, OFK_SCAN_FAST>), grid, block, 0, st, sc, bwd, post, T, N, stay, kSeries);
            else
                return OFK_BAD_ARGS;
            break;
        default: return OFK_BAD_ARGS;
    }
    return (int)hipGetLastError();
}

template <int S, int SPL, int DEPTH>
int launch_fused(int mode, const void *scores, float *bwd, float *post, int T, int N, float stay, hipStream_t st) {
    using Sh = FusedShape<S, SPL>;
    const dim3 grid((N + Sh::kChunks - 1) / Sh::kChunks), block(Sh::kThreads);
    const _Float16 *sc = static_cast<const _Float16 *>(scores);
    switch (mode) {
        case OFK_SCAN_TWO_TIER:
            hipLaunchKernelGGL((scan_post_kernel<S, SPL, DEPTH, OFK_SCAN_TWO_TIER>), grid, block, 0, st, sc, bwd, post, T, N, stay, kSeries);
            break;
        case OFK_SCAN_PRECISE:
            if constexpr (SPL == kPlainSpl<S>)
                hipLaunchKernelGGL((scan_post_kernel<S, SPL, DEPTH, OFK_SCAN_PRECISE>), grid, block, 0, st, sc, bwd, post, T, N, stay, kSeries);
            else
                return OFK_BAD_ARGS;
            break;
        case OFK_SCAN_FAST:
            if constexpr (SPL == kPlainSpl<S>)
                hipLaunchKernelGGL((scan_post_kernel<S, SPL, DEPTH, OFK_SCAN_FAST>), grid, block, 0, st, sc, bwd, post, T, N, stay, kSeries);
            else
                return OFK_BAD_ARGS;
            break;
        default: return OFK_BAD_ARGS;
    }
    return (int)hipGetLastError();
}

bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// States per lane: the largest of {4, 2, 1} (fewest lanes, least LDS traffic per state)
// that still gives every SIMD of the device (256 CUs x 4) a wave; small batches are
// spread thinner.  1024 states at one state per lane would need 1024-thread groups
// with a barrier per step, so that size stops at 2.
// The sweeps of the smaller models measure faster with two waves per SIMD (hac, 512 chunks:
// backward 1.29 ms against 1.33 ms; forward + posterior beside the beam search 1.41 ms against
// 1.61 ms, which is 13 000 chunks/s of a whole decode).
// `forced` = 4, 2 or 1 overrides the choice (0 = choose).
int states_per_lane(int S, int N, bool backward, int forced) {
    const int min_spl = S >= 1024 ? 2 : 1;
    if (forced == 4 || forced == 2 || forced == 1) return forced < min_spl ? min_spl : forced;
    const long wanted = S <= 256 ? 2048 : 1024;
    for (int spl = 4; spl > min_spl; spl >>= 1) {
        const long waves = ((long)N * (S / spl) + 63) / 64;
        if (waves >= wanted) return spl;
    }
    return min_spl;
}

}  // namespace

#ifndef OFK_DEPTH
#define OFK_DEPTH 8
#endif
#ifndef OFK_DEPTH_1024
#define OFK_DEPTH_1024 6
#endif
// The one-kernel scans keep the rows of two sweeps in flight.  Rows of one chunk lie N * C * 2 bytes
// apart; when that is a multiple of 4 MiB (2048 chunks of 256 states, 512 of 1024) all rows in
// flight fall onto the same DRAM banks, and with sixteen of them (eight per sweep) the kernel ran
// at half its rate and below (measured, 256 states, 2048 chunks: 8.97 ms; with four rows per sweep
// 5.69 ms, the rate of smaller batches; at 512 chunks both depths take 1.59 ms).  The separate
// sweeps, eight rows in flight altogether, never showed it.  Hence half the depth here.
#ifndef OFK_DEPTH_FUSED
#define OFK_DEPTH_FUSED 4
#endif
#ifndef OFK_DEPTH_FUSED_1024
#define OFK_DEPTH_FUSED_1024 3
#endif
#define OFK_DISPATCH(BACKWARD, LAUNCH, ...)                                                    \
    switch (state_len * 8 + states_per_lane(1 << (2 * state_len), N, BACKWARD, lanes_asked(mode, spl))) { \
        case 3 * 8 + 4: return LAUNCH<64, 4, OFK_DEPTH>(__VA_ARGS__);                          \
        case 3 * 8 + 2: return LAUNCH<64, 2, OFK_DEPTH>(__VA_ARGS__);                          \
        case 3 * 8 + 1: return LAUNCH<64, 1, OFK_DEPTH>(__VA_ARGS__);                          \
        case 4 * 8 + 4: return LAUNCH<256, 4, OFK_DEPTH>(__VA_ARGS__);                         \
        case 4 * 8 + 2: return LAUNCH<256, 2, OFK_DEPTH>(__VA_ARGS__);                         \
        case 4 * 8 + 1: return LAUNCH<256, 1, OFK_DEPTH>(__VA_ARGS__);                         \
        case 5 * 8 + 4: return LAUNCH<1024, 4, OFK_DEPTH_1024>(__VA_ARGS__);                        \
        case 5 * 8 + 2: return LAUNCH<1024, 2, OFK_DEPTH_1024>(__VA_ARGS__);                        \
        default: return OFK_BAD_ARGS;                                                  \
    }

// States per lane of the two-directional kernel: one direction of a chunk owns whole waves, so
// 64 states need one state per lane; as many lanes as it takes to put four waves on every SIMD,
// within the 1024 threads of a workgroup.
static int fused_states_per_lane(int S, int N, int forced) {
    const int min_spl = S >= 1024 ? 2 : 1, max_spl = S >= 256 ? 4 : 1;
    if (forced == 4 || forced == 2 || forced == 1) return forced < min_spl ? min_spl : (forced > max_spl ? max_spl : forced);
    for (int spl = max_spl; spl > min_spl; spl >>= 1) {
        const long waves = (long)N * 2 * (S / spl) / 64;
        if (waves >= 4096) return spl;
    }
    return min_spl;
}

// states per lane to force: the caller's wish (0 = none) with the default arithmetic, the fewest otherwise
static int lanes_asked(int mode, int spl) { return mode == OFK_SCAN_TWO_TIER ? spl : 1; }

static int scan_posterior(const void *scores, float *bwd, float *post, int T, int N, int state_len, float stay,
                          int mode, int spl, void *stream) {
    if (!scores || !bwd || !post || T < 1 || N < 1 || !aligned16(scores) || !aligned16(bwd) || !aligned16(post))
        return OFK_BAD_ARGS;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int S = 1 << (2 * state_len);
    switch (state_len * 8 + (state_len >= 3 && state_len <= 5 ? fused_states_per_lane(S, N, lanes_asked(mode, spl)) : 0)) {
        case 3 * 8 + 1:  // 64 states: latency-bound, the deeper prefetch pays until the rows are 4 MiB apart
            if ((size_t)N * kCols * S * 2 < ((size_t)4 << 20))
                return launch_fused<64, 1, OFK_DEPTH>(mode, scores, bwd, post, T, N, stay, st);
            return launch_fused<64, 1, OFK_DEPTH_FUSED>(mode, scores, bwd, post, T, N, stay, st);
        case 4 * 8 + 4: return launch_fused<256, 4, OFK_DEPTH_FUSED>(mode, scores, bwd, post, T, N, stay, st);
        case 4 * 8 + 2: return launch_fused<256, 2, OFK_DEPTH_FUSED>(mode, scores, bwd, post, T, N, stay, st);
        case 4 * 8 + 1: return launch_fused<256, 1, OFK_DEPTH_FUSED>(mode, scores, bwd, post, T, N, stay, st);
        case 5 * 8 + 4: return launch_fused<1024, 4, OFK_DEPTH_FUSED_1024>(mode, scores, bwd, post, T, N, stay, st);
        case 5 * 8 + 2: return launch_fused<1024, 2, OFK_DEPTH_FUSED_1024>(mode, scores, bwd, post, T, N, stay, st);
        default: return OFK_BAD_ARGS;
    }
}

static int bwd_scan(const void *scores, float *bwd, int T, int N, int state_len, float stay, int mode, int spl,
                    void *stream) {
    if (!scores || !bwd || T < 1 || N < 1 || !aligned16(scores) || !aligned16(bwd)) return OFK_BAD_ARGS;
    if (state_len < 3 || state_len > 5) return OFK_BAD_ARGS;
    hipStream_t st = static_cast<hipStream_t>(stream);
    OFK_DISPATCH(true, launch_bwd, mode, scores, bwd, T, N, stay, st)
}

static int fwd_post_scan(const void *scores, const float *bwd, float *post, int T, int N, int state_len,
                         float stay, int mode, int spl, void *stream) {
    if (!scores || !bwd || !post || T < 1 || N < 1 || !aligned16(scores) || !aligned16(bwd) || !aligned16(post))
        return OFK_BAD_ARGS;
    if (state_len < 3 || state_len > 5) return OFK_BAD_ARGS;
    hipStream_t st = static_cast<hipStream_t>(stream);
    OFK_DISPATCH(false, launch_fwd, mode, scores, bwd, post, T, N, stay, st)
}

// The build compiles this file twice: with four columns, which also holds the entry points, and
// with five, whose kernels the entry points reach through the three functions named *_five.
#if OFK_COLS == 5
extern "C" int ofk_scan_posterior_five(const void *scores, float *bwd, float *post, int T, int N, int state_len,
                                       float stay, int mode, int spl, void *stream) {
    return scan_posterior(scores, bwd, post, T, N, state_len, stay, mode, spl, stream);
}
extern "C" int ofk_bwd_scan_five(const void *scores, float *bwd, int T, int N, int state_len, float stay, int mode,
                                 int spl, void *stream) {
    return bwd_scan(scores, bwd, T, N, state_len, stay, mode, spl, stream);
}
extern "C" int ofk_fwd_post_scan_five(const void *scores, const float *bwd, float *post, int T, int N,
                                      int state_len, float stay, int mode, int spl, void *stream) {
    return fwd_post_scan(scores, bwd, post, T, N, state_len, stay, mode, spl, stream);
}
#else
extern "C" int ofk_scan_posterior_five(const void *, float *, float *, int, int, int, float, int, int, void *);
extern "C" int ofk_bwd_scan_five(const void *, float *, int, int, int, float, int, int, void *);
extern "C" int ofk_fwd_post_scan_five(const void *, const float *, float *, int, int, int, float, int, int, void *);

extern "C" int ofk_scan_posterior(const void *scores, float *bwd, float *post, int T, int N, int state_len,
                                  int columns, float stay, int mode, int spl, void *stream) {
    if (columns == 5) return ofk_scan_posterior_five(scores, bwd, post, T, N, state_len, stay, mode, spl, stream);
    if (columns != 4) return OFK_BAD_ARGS;
    return scan_posterior(scores, bwd, post, T, N, state_len, stay, mode, spl, stream);
}

extern "C" int ofk_bwd_scan(const void *scores, float *bwd, int T, int N, int state_len, int columns, float stay,
                            int mode, int spl, void *stream) {
    if (columns == 5) return ofk_bwd_scan_five(scores, bwd, T, N, state_len, stay, mode, spl, stream);
    if (columns != 4) return OFK_BAD_ARGS;
    return bwd_scan(scores, bwd, T, N, state_len, stay, mode, spl, stream);
}

extern "C" int ofk_fwd_post_scan(const void *scores, const float *bwd, float *post, int T, int N, int state_len,
                                 int columns, float stay, int mode, int spl, void *stream) {
    if (columns == 5) return ofk_fwd_post_scan_five(scores, bwd, post, T, N, state_len, stay, mode, spl, stream);
    if (columns != 4) return OFK_BAD_ARGS;
    return fwd_post_scan(scores, bwd, post, T, N, state_len, stay, mode, spl, stream);
}
#endif
