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
// in transition order, max + log(sum).  Two variants of that last step exist:
//   precise: exp and log in double, the running sum rounded to fp32 after every
//            term and one rounding of max + log(sum), i.e. the CPU path's own
//            sequence of roundings (fp64 FMA issues at the fp32 rate on gfx950);
//   fast   : v_exp_f32 / v_log_f32, within an ulp or two of the precise result.
// State values reach several thousand, where one fp32 ulp is already 5e-4, and
// the posterior is exp(fwd + bwd - const): a last-bit difference in a scan shows
// up as a 5e-4 relative difference of a posterior.  The precise variant is the
// default for that reason.
#include <hip/hip_runtime.h>

#include "dmath.h"
#include "kernels.h"

namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));

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

// What the CPU-faithful logarithm reads: its table in LDS and its series coefficients.  The
// coefficients travel as a kernel argument, which puts them into scalar registers for the whole
// kernel (as literals the compiler copies them into vector registers at every use).
struct LogSeries {
    double c[6];
};
struct LogArgs {
    const ofa::LogCell *cells;
    const double *series;
};

// max + log(sum_i exp(v_i - max)), sum taken in the order v0..v4
template <bool PRECISE>
__device__ __forceinline__ float lse5(float v0, float v1, float v2, float v3, float v4, const LogArgs &logtab) {
    const float m = fmaxf(fmaxf(fmaxf(v0, v1), v2), fmaxf(v3, v4));
    if constexpr (PRECISE) {
        return ofa::lse5_cpu_rounding_tab(v0, v1, v2, v3, v4, m, logtab.cells, logtab.series);
    } else {
        float s = __builtin_amdgcn_exp2f((v0 - m) * kLog2e);
        s += __builtin_amdgcn_exp2f((v1 - m) * kLog2e);
        s += __builtin_amdgcn_exp2f((v2 - m) * kLog2e);
        s += __builtin_amdgcn_exp2f((v3 - m) * kLog2e);
        s += __builtin_amdgcn_exp2f((v4 - m) * kLog2e);
        return __builtin_fmaf(__builtin_amdgcn_logf(s), kLn2, m);
    }
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

// The scores one lane needs for one time step, as loaded (fp16).
// Backward: transition b of own state i is element 4b + i of the lane's window.
template <int SPL>
struct BwdRow;
template <>
struct BwdRow<4> {
    half8 v[2];
    __device__ __forceinline__ void load(const _Float16 *p) {
        v[0] = reinterpret_cast<const half8 *>(p)[0];
        v[1] = reinterpret_cast<const half8 *>(p)[1];
    }
    template <int B, int I>
    __device__ __forceinline__ float get() const { return (float)v[(4 * B + I) / 8][(4 * B + I) % 8]; }
};
template <>
struct BwdRow<2> {
    half2v v[4];
    __device__ __forceinline__ void load(const _Float16 *p) {
#pragma unroll
        for (int b = 0; b < 4; ++b) v[b] = *reinterpret_cast<const half2v *>(p + 4 * b);
    }
    template <int B, int I>
    __device__ __forceinline__ float get() const { return (float)v[B][I]; }
};
template <>
struct BwdRow<1> {
    _Float16 v[4];
    __device__ __forceinline__ void load(const _Float16 *p) {
#pragma unroll
        for (int b = 0; b < 4; ++b) v[b] = p[4 * b];
    }
    template <int B, int I>
    __device__ __forceinline__ float get() const { return (float)v[B]; }
};

// Forward: transition b into own state i is element 4i + b of the lane's window.
template <int SPL>
struct FwdRow;
template <>
struct FwdRow<4> {
    half8 v[2];
    __device__ __forceinline__ void load(const _Float16 *p) {
        v[0] = reinterpret_cast<const half8 *>(p)[0];
        v[1] = reinterpret_cast<const half8 *>(p)[1];
    }
    template <int I, int B>
    __device__ __forceinline__ float get() const { return (float)v[(4 * I + B) / 8][(4 * I + B) % 8]; }
};
template <>
struct FwdRow<2> {
    half8 v;
    __device__ __forceinline__ void load(const _Float16 *p) { v = *reinterpret_cast<const half8 *>(p); }
    template <int I, int B>
    __device__ __forceinline__ float get() const { return (float)v[4 * I + B]; }
};
template <>
struct FwdRow<1> {
    half4 v;
    __device__ __forceinline__ void load(const _Float16 *p) { v = *reinterpret_cast<const half4 *>(p); }
    template <int I, int B>
    __device__ __forceinline__ float get() const { return (float)v[B]; }
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

template <int I, int SPL, bool PRECISE>
__device__ __forceinline__ void bwd_update(float (&a)[SPL], const float4 &nx, const BwdRow<SPL> &row, float stay,
                                           const LogArgs &logtab) {
    if constexpr (I < SPL) {
        a[I] = lse5<PRECISE>(a[I] + stay, nx.x + row.template get<0, I>(), nx.y + row.template get<1, I>(),
                             nx.z + row.template get<2, I>(), nx.w + row.template get<3, I>(), logtab);
        bwd_update<I + 1, SPL, PRECISE>(a, nx, row, stay, logtab);
    }
}

template <int I, int SPL, bool PRECISE>
__device__ __forceinline__ void fwd_update(float (&f)[SPL], float p0, float p1, float p2, float p3,
                                           const FwdRow<SPL> &row, float stay, const LogArgs &logtab) {
    if constexpr (I < SPL) {
        f[I] = lse5<PRECISE>(f[I] + stay, p0 + row.template get<I, 0>(), p1 + row.template get<I, 1>(),
                             p2 + row.template get<I, 2>(), p3 + row.template get<I, 3>(), logtab);
        fwd_update<I + 1, SPL, PRECISE>(f, p0, p1, p2, p3, row, stay, logtab);
    }
}

// ---------------------------------------------------------------------------
// backward: bwd[n][t][s] for t = T..0
// ---------------------------------------------------------------------------
template <int S, int SPL, int DEPTH, bool PRECISE>
__global__ __launch_bounds__((Shape<S, SPL>::kThreads)) void bwd_scan_kernel(
    const _Float16 *__restrict__ scores, float *__restrict__ bwd, int T, int N, float stay, LogSeries series) {
    using Sh = Shape<S, SPL>;
    constexpr int L = Sh::kLanes;
    constexpr int Q = Sh::kQuarter;
    constexpr int H = 4 / SPL;  // lanes sharing one quad
    __shared__ __attribute__((aligned(16))) float vec[Sh::kChunks][2][S];
    __shared__ __attribute__((aligned(16))) ofa::LogCell logcells[32];
    const LogArgs logtab{logcells, series.c};

    const int tid = threadIdx.x;
    if (PRECISE && tid < 32) logcells[tid] = ofa::log_cell(tid);
    const int g = tid / L, l = tid % L;
    const int r = l / H, c0 = (l % H) * SPL;  // own states: r + (c0 + i) * Q
    int n = blockIdx.x * Sh::kChunks + g;
    const bool live = n < N;
    if (!live) n = N - 1;

    const size_t row_stride = (size_t)N * 4 * S;  // fp16 elements between time steps
    const _Float16 *sp = scores + (size_t)n * 4 * S + 16 * r + c0;
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
    for (int i = 0; i < SPL; ++i) vec[g][0][r + (c0 + i) * Q] = 0.f;
    __syncthreads();  // the log table is shared by the whole group

    for (int done = 0; done < T; done += DEPTH) {
#pragma unroll
        for (int k = 0; k < DEPTH; ++k) {
            const int t = T - 1 - done - k;
            if (t >= 0) {
                const BwdRow<SPL> row = ring[k];
                if (t - DEPTH >= 0) ring[k].load(sp + (size_t)(t - DEPTH) * row_stride);
                chunk_sync<Sh::kMultiWave>();
                const float4 nx = *reinterpret_cast<const float4 *>(&vec[g][buf][4 * r]);
                bwd_update<0, SPL, PRECISE>(a, nx, row, stay, logtab);
                buf ^= 1;
#pragma unroll
                for (int i = 0; i < SPL; ++i) vec[g][buf][r + (c0 + i) * Q] = a[i];
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
template <int S, int SPL, int DEPTH, bool PRECISE>
__global__ __launch_bounds__((Shape<S, SPL>::kThreads)) void fwd_post_kernel(
    const _Float16 *__restrict__ scores, const float *__restrict__ bwd, float *__restrict__ post, int T,
    int N, float stay, LogSeries series) {
    using Sh = Shape<S, SPL>;
    constexpr int L = Sh::kLanes;
    constexpr int Q = Sh::kQuarter;
    __shared__ __attribute__((aligned(16))) float vec[Sh::kChunks][2][S];
    __shared__ float part[2][Sh::kChunks][Sh::kChunkWaves];
    __shared__ __attribute__((aligned(16))) ofa::LogCell logcells[32];
    const LogArgs logtab{logcells, series.c};

    const int tid = threadIdx.x;
    if (PRECISE && tid < 32) logcells[tid] = ofa::log_cell(tid);
    const int g = tid / L, l = tid % L;
    const int s0 = SPL * l, q = s0 >> 2;  // own states s0 .. s0+SPL-1, all in quad q
    const int wave = l / 64;  // wave within the chunk
    int n = blockIdx.x * Sh::kChunks + g;
    const bool live = n < N;
    if (!live) n = N - 1;

    const size_t row_stride = (size_t)N * 4 * S;
    const _Float16 *sp = scores + (size_t)n * 4 * S + 4 * s0;
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
                    fwd_update<0, SPL, PRECISE>(f, p0, p1, p2, p3, row, stay, logtab);
                    buf ^= 1;
                }
            }
        }
    }
}

int g_scan_fast = 0;
int g_scan_spl = 0;  // 0 = choose from the batch size

const LogSeries kSeries = {OFA_LOG_SERIES};

template <int S, int SPL, int DEPTH>
int launch_bwd(const void *scores, float *bwd, int T, int N, float stay, hipStream_t st) {
    using Sh = Shape<S, SPL>;
    const int blocks = (N + Sh::kChunks - 1) / Sh::kChunks;
    if (g_scan_fast)
        hipLaunchKernelGGL((bwd_scan_kernel<S, SPL, DEPTH, false>), dim3(blocks), dim3(Sh::kThreads), 0, st,
                           static_cast<const _Float16 *>(scores), bwd, T, N, stay, kSeries);
    else
        hipLaunchKernelGGL((bwd_scan_kernel<S, SPL, DEPTH, true>), dim3(blocks), dim3(Sh::kThreads), 0, st,
                           static_cast<const _Float16 *>(scores), bwd, T, N, stay, kSeries);
    return (int)hipGetLastError();
}

template <int S, int SPL, int DEPTH>
int launch_fwd(const void *scores, const float *bwd, float *post, int T, int N, float stay, hipStream_t st) {
    using Sh = Shape<S, SPL>;
    const int blocks = (N + Sh::kChunks - 1) / Sh::kChunks;
    if (g_scan_fast)
        hipLaunchKernelGGL((fwd_post_kernel<S, SPL, DEPTH, false>), dim3(blocks), dim3(Sh::kThreads), 0, st,
                           static_cast<const _Float16 *>(scores), bwd, post, T, N, stay, kSeries);
    else
        hipLaunchKernelGGL((fwd_post_kernel<S, SPL, DEPTH, true>), dim3(blocks), dim3(Sh::kThreads), 0, st,
                           static_cast<const _Float16 *>(scores), bwd, post, T, N, stay, kSeries);
    return (int)hipGetLastError();
}

bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// States per lane: the largest of {4, 2, 1} (fewest lanes, least LDS traffic per state)
// that still gives every SIMD of the device (256 CUs x 4) a wave; small batches are
// spread thinner.  1024 states at one state per lane would need 1024-thread groups
// with a barrier per step, so that size stops at 2.
// The backward sweep of the smaller models measures faster with two waves per SIMD
// (hac, 512 chunks: 1.29 ms against 1.33 ms; 0.56 against 0.68 ms with hardware exp/log).
int states_per_lane(int S, int N, bool backward) {
    const int min_spl = S >= 1024 ? 2 : 1;
    if (g_scan_spl == 4 || g_scan_spl == 2 || g_scan_spl == 1) return g_scan_spl < min_spl ? min_spl : g_scan_spl;
    const long wanted = (backward && S <= 256) ? 2048 : 1024;
    for (int spl = 4; spl > min_spl; spl >>= 1) {
        const long waves = ((long)N * (S / spl) + 63) / 64;
        if (waves >= wanted) return spl;
    }
    return min_spl;
}

}  // namespace

extern "C" void ofk_set_scan_fast(int on) { g_scan_fast = on; }
extern "C" void ofk_set_scan_states_per_lane(int spl) { g_scan_spl = spl; }

#define OFK_DISPATCH(BACKWARD, LAUNCH, ...)                                                    \
    switch (state_len * 8 + states_per_lane(1 << (2 * state_len), N, BACKWARD)) {             \
        case 3 * 8 + 4: return LAUNCH<64, 4, 8>(__VA_ARGS__);                          \
        case 3 * 8 + 2: return LAUNCH<64, 2, 8>(__VA_ARGS__);                          \
        case 3 * 8 + 1: return LAUNCH<64, 1, 8>(__VA_ARGS__);                          \
        case 4 * 8 + 4: return LAUNCH<256, 4, 8>(__VA_ARGS__);                         \
        case 4 * 8 + 2: return LAUNCH<256, 2, 8>(__VA_ARGS__);                         \
        case 4 * 8 + 1: return LAUNCH<256, 1, 8>(__VA_ARGS__);                         \
        case 5 * 8 + 4: return LAUNCH<1024, 4, 6>(__VA_ARGS__);                        \
        case 5 * 8 + 2: return LAUNCH<1024, 2, 6>(__VA_ARGS__);                        \
        default: return OFK_BAD_ARGS;                                                  \
    }

extern "C" int ofk_bwd_scan(const void *scores, float *bwd, int T, int N, int state_len, float stay,
                            void *stream) {
    if (!scores || !bwd || T < 1 || N < 1 || !aligned16(scores) || !aligned16(bwd)) return OFK_BAD_ARGS;
    if (state_len < 3 || state_len > 5) return OFK_BAD_ARGS;
    hipStream_t st = static_cast<hipStream_t>(stream);
    OFK_DISPATCH(true, launch_bwd, scores, bwd, T, N, stay, st)
}

extern "C" int ofk_fwd_post_scan(const void *scores, const float *bwd, float *post, int T, int N,
                                 int state_len, float stay, void *stream) {
    if (!scores || !bwd || !post || T < 1 || N < 1 || !aligned16(scores) || !aligned16(bwd) || !aligned16(post))
        return OFK_BAD_ARGS;
    if (state_len < 3 || state_len > 5) return OFK_BAD_ARGS;
    hipStream_t st = static_cast<hipStream_t>(stream);
    OFK_DISPATCH(false, launch_fwd, scores, bwd, post, T, N, stay, st)
}
