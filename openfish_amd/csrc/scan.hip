// Backward and forward log-space scans over the 4^state_len CRF states, gfx950.
//
// The k-mer transition graph has a quad structure: the four states {4q+j} share
// the four predecessors {q + b*S/4} and the 16 contiguous scores [16q, 16q+16)
// (element 4j+b is the transition pred b -> state 4q+j).  A lane owns one quad:
//   forward : owns the contiguous quad {4q+j}, needs the strided quad of the
//             previous vector (4 LDS reads), its own values stay in registers;
//   backward: owns the strided quad {r + c*S/4}, needs the contiguous quad
//             {4r+b} of the next vector (one 128-bit LDS read).
// Per time step a lane therefore reads 32 contiguous bytes of fp16 scores (a
// wave reads one 2 KB row segment, fully coalesced), exchanges the state vector
// through LDS and, when a chunk fits one wavefront, needs no block barrier.
// Score rows (and bwd rows in the forward sweep) for the next DEPTH time steps
// are kept in flight in registers.
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

#include "kernels.h"

namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));

constexpr float kLog2e = 1.44269504088896340736f;
constexpr float kLn2 = 0.69314718055994530942f;

template <int CTRL>
__device__ __forceinline__ float dpp(float x) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xF, 0xF, true));
}
__device__ __forceinline__ float lane_value(float x, int lane) {
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(x), lane));
}

// reductions over the lanes of one chunk inside a wave: LANES is 16 (one DPP row)
// or 64 (whole wave).  Every lane of the group ends with the same bits.
template <int LANES>
__device__ __forceinline__ float group_sum(float x) {
    x += dpp<0x128>(x);  // row_ror:8
    x += dpp<0x124>(x);  // row_ror:4
    x += dpp<0x122>(x);  // row_ror:2
    x += dpp<0x121>(x);  // row_ror:1
    if constexpr (LANES >= 64) {
        x = (lane_value(x, 0) + lane_value(x, 16)) + (lane_value(x, 32) + lane_value(x, 48));
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
    }
    return x;
}

// max + log(sum_i exp(v_i - max)), sum taken in the order v0..v4
template <bool PRECISE>
__device__ __forceinline__ float lse5(float v0, float v1, float v2, float v3, float v4) {
    const float m = fmaxf(fmaxf(fmaxf(v0, v1), v2), fmaxf(v3, v4));
    if constexpr (PRECISE) {
        float s = (float)exp((double)(v0 - m));
        s = (float)((double)s + exp((double)(v1 - m)));
        s = (float)((double)s + exp((double)(v2 - m)));
        s = (float)((double)s + exp((double)(v3 - m)));
        s = (float)((double)s + exp((double)(v4 - m)));
        return (float)((double)m + log((double)s));
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
        __syncthreads();
    } else {
        // one wavefront per chunk: LDS operations of a wave complete in order, only the
        // compiler has to be kept from moving the reads above the writes
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
}

template <int S>
struct Shape {
    static constexpr int kLanes = S / 4;                           // lanes per chunk
    static constexpr int kChunks = kLanes >= 64 ? 1 : 64 / kLanes;  // chunks per workgroup
    static constexpr int kThreads = kLanes >= 64 ? kLanes : 64;
    static constexpr bool kMultiWave = kLanes > 64;
    static constexpr int kGroup = kLanes >= 64 ? 64 : kLanes;       // chunk lanes inside one wave
    static constexpr int kWaves = kThreads / 64;
};

// ---------------------------------------------------------------------------
// backward: bwd[n][t][s] for t = T..0
// ---------------------------------------------------------------------------
template <int S, int DEPTH, bool PRECISE>
__global__ __launch_bounds__(Shape<S>::kThreads) void bwd_scan_kernel(
    const _Float16 *__restrict__ scores, float *__restrict__ bwd, int T, int N, float stay) {
    using Sh = Shape<S>;
    constexpr int L = Sh::kLanes;
    __shared__ __attribute__((aligned(16))) float vec[Sh::kChunks][2][S];

    const int tid = threadIdx.x;
    const int g = tid / L, r = tid % L;
    int n = blockIdx.x * Sh::kChunks + g;
    const bool live = n < N;
    if (!live) n = N - 1;

    const size_t row_stride = (size_t)N * 4 * S;  // fp16 elements between time steps
    const _Float16 *sp = scores + (size_t)n * 4 * S + 16 * r;
    float *out = bwd + (size_t)n * (size_t)(T + 1) * S + r;

    float a[4] = {0.f, 0.f, 0.f, 0.f};  // values of states r + c*L
    if (live) {
#pragma unroll
        for (int c = 0; c < 4; ++c) out[(size_t)T * S + c * L] = 0.f;
    }

    half8 ring[DEPTH][2];
#pragma unroll
    for (int k = 0; k < DEPTH; ++k) {
        const int t = T - 1 - k;
        if (t >= 0) {
            const half8 *p = reinterpret_cast<const half8 *>(sp + (size_t)t * row_stride);
            ring[k][0] = p[0];
            ring[k][1] = p[1];
        }
    }

    int buf = 0;
#pragma unroll
    for (int c = 0; c < 4; ++c) vec[g][0][r + c * L] = 0.f;

    for (int done = 0; done < T; done += DEPTH) {
#pragma unroll
        for (int k = 0; k < DEPTH; ++k) {
            const int t = T - 1 - done - k;
            if (t >= 0) {
                const half8 lo = ring[k][0], hi = ring[k][1];
                if (t - DEPTH >= 0) {
                    const half8 *p = reinterpret_cast<const half8 *>(sp + (size_t)(t - DEPTH) * row_stride);
                    ring[k][0] = p[0];
                    ring[k][1] = p[1];
                }
                chunk_sync<Sh::kMultiWave>();
                const float4 nx = *reinterpret_cast<const float4 *>(&vec[g][buf][4 * r]);
                // score of the transition (r + c*L) -> (4r + b) sits at 4b + c
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    const float v0 = a[c] + stay;
                    const float v1 = nx.x + (float)lo[c];
                    const float v2 = nx.y + (float)lo[4 + c];
                    const float v3 = nx.z + (float)hi[c];
                    const float v4 = nx.w + (float)hi[4 + c];
                    a[c] = lse5<PRECISE>(v0, v1, v2, v3, v4);
                }
                buf ^= 1;
#pragma unroll
                for (int c = 0; c < 4; ++c) vec[g][buf][r + c * L] = a[c];
                if (live) {
#pragma unroll
                    for (int c = 0; c < 4; ++c) out[(size_t)t * S + c * L] = a[c];
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------
// forward + posterior: post[n][t][s] = softmax_s(fwd[t][s] + bwd[n][t][s]), t = 0..T
// ---------------------------------------------------------------------------
template <int S, int DEPTH, bool PRECISE>
__global__ __launch_bounds__(Shape<S>::kThreads) void fwd_post_kernel(
    const _Float16 *__restrict__ scores, const float *__restrict__ bwd, float *__restrict__ post, int T,
    int N, float stay) {
    using Sh = Shape<S>;
    constexpr int L = Sh::kLanes;
    __shared__ __attribute__((aligned(16))) float vec[Sh::kChunks][2][S];
    __shared__ float part[2][Sh::kWaves];

    const int tid = threadIdx.x;
    const int g = tid / L, q = tid % L;
    const int wave = tid / 64;
    int n = blockIdx.x * Sh::kChunks + g;
    const bool live = n < N;
    if (!live) n = N - 1;

    const size_t row_stride = (size_t)N * 4 * S;
    const _Float16 *sp = scores + (size_t)n * 4 * S + 16 * q;
    const float *bp = bwd + (size_t)n * (size_t)(T + 1) * S + 4 * q;
    float *pp = post + (size_t)n * (size_t)(T + 1) * S + 4 * q;

    half8 ring[DEPTH][2];
    float4 bring[DEPTH];
#pragma unroll
    for (int k = 0; k < DEPTH; ++k) {
        if (k < T) {
            const half8 *p = reinterpret_cast<const half8 *>(sp + (size_t)k * row_stride);
            ring[k][0] = p[0];
            ring[k][1] = p[1];
        }
        if (k <= T) bring[k] = *reinterpret_cast<const float4 *>(bp + (size_t)k * S);
    }

    // Shift of the softmax exponent.  sum_s exp(fwd+bwd) is the same partition function at
    // every time step, and at t = 0 it lies within log(S) of max_s bwd[0][s]; that maximum,
    // lowered by 10 so that tiny posteriors stay normal numbers until the final product,
    // replaces the per-step maximum (the quotient does not depend on the shift).
    float shift;
    {
        const float4 b0 = *reinterpret_cast<const float4 *>(bp);
        float m = group_max<Sh::kGroup>(fmaxf(fmaxf(b0.x, b0.y), fmaxf(b0.z, b0.w)));
        if constexpr (Sh::kMultiWave) {
            if ((tid & 63) == 0) part[0][wave] = m;
            __syncthreads();
            m = part[0][0];
#pragma unroll
            for (int w = 1; w < Sh::kWaves; ++w) m = fmaxf(m, part[0][w]);
            __syncthreads();
        }
        shift = m - 10.0f;
    }

    float f[4] = {0.f, 0.f, 0.f, 0.f};  // values of states 4q + j
    int buf = 0;

    for (int done = 0; done <= T; done += DEPTH) {
#pragma unroll
        for (int k = 0; k < DEPTH; ++k) {
            const int t = done + k;
            if (t <= T) {
                const half8 lo = ring[k][0], hi = ring[k][1];
                const float4 bw = bring[k];
                if (t + DEPTH < T) {
                    const half8 *p = reinterpret_cast<const half8 *>(sp + (size_t)(t + DEPTH) * row_stride);
                    ring[k][0] = p[0];
                    ring[k][1] = p[1];
                }
                if (t + DEPTH <= T) bring[k] = *reinterpret_cast<const float4 *>(bp + (size_t)(t + DEPTH) * S);

                // posterior of time step t
                float e0 = __builtin_amdgcn_exp2f(((f[0] + bw.x) - shift) * kLog2e);
                float e1 = __builtin_amdgcn_exp2f(((f[1] + bw.y) - shift) * kLog2e);
                float e2 = __builtin_amdgcn_exp2f(((f[2] + bw.z) - shift) * kLog2e);
                float e3 = __builtin_amdgcn_exp2f(((f[3] + bw.w) - shift) * kLog2e);
                float total = group_sum<Sh::kGroup>((e0 + e1) + (e2 + e3));

                *reinterpret_cast<float4 *>(&vec[g][buf][4 * q]) = make_float4(f[0], f[1], f[2], f[3]);
                if constexpr (Sh::kMultiWave) {
                    if ((tid & 63) == 0) part[buf][wave] = total;
                }
                chunk_sync<Sh::kMultiWave>();
                if constexpr (Sh::kMultiWave) {
                    total = part[buf][0];
#pragma unroll
                    for (int w = 1; w < Sh::kWaves; ++w) total += part[buf][w];
                }
                const float inv = __builtin_amdgcn_rcpf(total);
                if (live) *reinterpret_cast<float4 *>(pp + (size_t)t * S) = make_float4(e0 * inv, e1 * inv, e2 * inv, e3 * inv);

                if (t < T) {
                    const float p0 = vec[g][buf][q];
                    const float p1 = vec[g][buf][q + L];
                    const float p2 = vec[g][buf][q + 2 * L];
                    const float p3 = vec[g][buf][q + 3 * L];
                    // score of the transition (q + b*L) -> (4q + j) sits at 4j + b
                    f[0] = lse5<PRECISE>(f[0] + stay, p0 + (float)lo[0], p1 + (float)lo[1], p2 + (float)lo[2], p3 + (float)lo[3]);
                    f[1] = lse5<PRECISE>(f[1] + stay, p0 + (float)lo[4], p1 + (float)lo[5], p2 + (float)lo[6], p3 + (float)lo[7]);
                    f[2] = lse5<PRECISE>(f[2] + stay, p0 + (float)hi[0], p1 + (float)hi[1], p2 + (float)hi[2], p3 + (float)hi[3]);
                    f[3] = lse5<PRECISE>(f[3] + stay, p0 + (float)hi[4], p1 + (float)hi[5], p2 + (float)hi[6], p3 + (float)hi[7]);
                    buf ^= 1;
                }
            }
        }
    }
}

int g_scan_fast = 0;

template <int S, int DEPTH>
int launch_bwd(const void *scores, float *bwd, int T, int N, float stay, hipStream_t st) {
    using Sh = Shape<S>;
    const int blocks = (N + Sh::kChunks - 1) / Sh::kChunks;
    if (g_scan_fast)
        hipLaunchKernelGGL((bwd_scan_kernel<S, DEPTH, false>), dim3(blocks), dim3(Sh::kThreads), 0, st,
                           static_cast<const _Float16 *>(scores), bwd, T, N, stay);
    else
        hipLaunchKernelGGL((bwd_scan_kernel<S, DEPTH, true>), dim3(blocks), dim3(Sh::kThreads), 0, st,
                           static_cast<const _Float16 *>(scores), bwd, T, N, stay);
    return (int)hipGetLastError();
}

template <int S, int DEPTH>
int launch_fwd(const void *scores, const float *bwd, float *post, int T, int N, float stay, hipStream_t st) {
    using Sh = Shape<S>;
    const int blocks = (N + Sh::kChunks - 1) / Sh::kChunks;
    if (g_scan_fast)
        hipLaunchKernelGGL((fwd_post_kernel<S, DEPTH, false>), dim3(blocks), dim3(Sh::kThreads), 0, st,
                           static_cast<const _Float16 *>(scores), bwd, post, T, N, stay);
    else
        hipLaunchKernelGGL((fwd_post_kernel<S, DEPTH, true>), dim3(blocks), dim3(Sh::kThreads), 0, st,
                           static_cast<const _Float16 *>(scores), bwd, post, T, N, stay);
    return (int)hipGetLastError();
}

bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

}  // namespace

extern "C" void ofk_set_scan_fast(int on) { g_scan_fast = on; }

extern "C" int ofk_bwd_scan(const void *scores, float *bwd, int T, int N, int state_len, float stay,
                            void *stream) {
    if (!scores || !bwd || T < 1 || N < 1 || !aligned16(scores) || !aligned16(bwd)) return OFK_BAD_ARGS;
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (state_len) {
        case 3: return launch_bwd<64, 8>(scores, bwd, T, N, stay, st);
        case 4: return launch_bwd<256, 8>(scores, bwd, T, N, stay, st);
        case 5: return launch_bwd<1024, 6>(scores, bwd, T, N, stay, st);
        default: return OFK_BAD_ARGS;
    }
}

extern "C" int ofk_fwd_post_scan(const void *scores, const float *bwd, float *post, int T, int N,
                                 int state_len, float stay, void *stream) {
    if (!scores || !bwd || !post || T < 1 || N < 1 || !aligned16(scores) || !aligned16(bwd) || !aligned16(post))
        return OFK_BAD_ARGS;
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (state_len) {
        case 3: return launch_fwd<64, 8>(scores, bwd, post, T, N, stay, st);
        case 4: return launch_fwd<256, 8>(scores, bwd, post, T, N, stay, st);
        case 5: return launch_fwd<1024, 6>(scores, bwd, post, T, N, stay, st);
        default: return OFK_BAD_ARGS;
    }
}
