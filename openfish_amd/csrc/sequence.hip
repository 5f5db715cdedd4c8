// Per-block quality, base calls and phred characters of one chunk per workgroup, gfx950.
//
// Follows the CPU path (reference src/beam_search.c:441-496 for the quality of a
// block, src/beam_search.c:49-99 and src/decode_cpu.c:218-225 for the sequence):
//   1. every time step in parallel: posterior of the path k-mer plus its distinct
//      one-base shifts (fp32 sums in the CPU path's order), clamped, to the power 0.4;
//   2. a block-wide prefix sum of the moves gives every time step its base position;
//   3. every base in parallel: the fp32 sums over its dwell are taken in time order,
//      exactly as the serial loop takes them, then the phred character follows.
// pow is evaluated in double and rounded once to fp32.  The phred character is a
// step function of the miss probability 1 - base/total; its 49 thresholds are
// found on the host with the host's own log10f and handed in, so the character
// does not depend on a device log10.
#include <hip/hip_runtime.h>

#include "kernels.h"

namespace {

constexpr int kThreads = 256;

template <int S>
__global__ __launch_bounds__(kThreads) void sequence_kernel(
    const float *__restrict__ post, int32_t *__restrict__ states, const uint8_t *__restrict__ moves,
    float *__restrict__ qual_data, float *__restrict__ base_probs, float *__restrict__ total_probs,
    char *__restrict__ sequence, char *__restrict__ qstring, int T, ofk_phred_table_t phred) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    float *s_prob = reinterpret_cast<float *>(lds);        // [T] called-base probability
    float *s_wrong = s_prob + T;                           // [T] probability of each other base
    int *s_start = reinterpret_cast<int *>(s_wrong + T);   // [T+1] first time step of base p
    unsigned char *s_base = reinterpret_cast<unsigned char *>(s_start + T + 1);  // [T]
    unsigned char *s_move = s_base + T;                    // [T]
    __shared__ int s_scan[kThreads];

    const int n = blockIdx.x;
    const int tid = threadIdx.x;
    const float *post_n = post + (size_t)n * (size_t)(T + 1) * S;
    int32_t *st_n = states + (size_t)n * T;
    const uint8_t *mv_n = moves + (size_t)n * T;

    // 1. quality of every block
    for (int t = tid; t < T; t += kThreads) {
        const int st = st_n[t];
        const int base = st & 3;
        st_n[t] = base;
        const float *p = post_n + (size_t)(t + 1) * S;
        float prob = p[st];
        int nb[8];
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            nb[2 * b] = (st >> 2) + (S / 4) * b;
            nb[2 * b + 1] = ((st << 2) & (S - 1)) + b;
        }
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            bool fresh = nb[k] != st;
#pragma unroll
            for (int m = 0; m < k; ++m) fresh = fresh && nb[m] != nb[k];
            if (fresh) prob += p[nb[k]];
        }
        if (prob > 1.0f) prob = 1.0f;
        else if (prob < 0.0f) prob = 0.0f;
        prob = (float)pow((double)prob, (double)0.4f);
        const float wrong = (1.0f - prob) / 3.0f;
        s_prob[t] = prob;
        s_wrong[t] = wrong;
        s_base[t] = (unsigned char)base;
        s_move[t] = mv_n[t];
        float4 q;
        q.x = base == 0 ? prob : wrong;
        q.y = base == 1 ? prob : wrong;
        q.z = base == 2 ? prob : wrong;
        q.w = base == 3 ? prob : wrong;
        reinterpret_cast<float4 *>(qual_data)[(size_t)n * T + t] = q;
    }
    __syncthreads();

    // 2. base position of every time step: inclusive prefix sum of the moves, minus one
    const int seg = (T + kThreads - 1) / kThreads;
    const int t_lo = tid * seg < T ? tid * seg : T;
    const int t_hi = t_lo + seg < T ? t_lo + seg : T;
    int mine = 0;
    for (int t = t_lo; t < t_hi; ++t) mine += s_move[t];
    s_scan[tid] = mine;
    __syncthreads();
    for (int d = 1; d < kThreads; d <<= 1) {
        const int add = tid >= d ? s_scan[tid - d] : 0;
        __syncthreads();
        s_scan[tid] += add;
        __syncthreads();
    }
    const int seq_len = s_scan[kThreads - 1];
    {
        int pos = s_scan[tid] - mine;  // bases emitted before this segment
        for (int t = t_lo; t < t_hi; ++t) {
            if (s_move[t]) s_start[pos++] = t;
        }
        if (tid == 0) s_start[seq_len] = T;
    }
    __syncthreads();

    // 3. one base per thread
    for (int p = tid; p < T; p += kThreads) {
        const size_t o = (size_t)n * T + p;
        if (p >= seq_len) {
            sequence[o] = 0;
            qstring[o] = 0;
            base_probs[o] = 0.f;
            total_probs[o] = 0.f;
            continue;
        }
        const int t0 = s_start[p], t1 = s_start[p + 1];
        float bp = 0.f, tp = 0.f;
        for (int t = t0; t < t1; ++t) {
            const float prob = s_prob[t], wrong = s_wrong[t];
            const int base = s_base[t];
            bp += prob;
            tp += base == 0 ? prob : wrong;
            tp += base == 1 ? prob : wrong;
            tp += base == 2 ? prob : wrong;
            tp += base == 3 ? prob : wrong;
        }
        const float miss = 1.0f - (bp / tp);
        int ch = 83;
#pragma unroll
        for (int j = 0; j < OFK_PHRED_STEPS; ++j) ch -= miss >= phred.thr[j] ? 1 : 0;
        if (miss != miss) ch = 0;
        sequence[o] = "ACGT"[s_base[t0]];
        qstring[o] = (char)ch;
        base_probs[o] = -10.0f * (float)log10((double)miss);  // diagnostic copy, not used for the character
        total_probs[o] = tp;
    }
}

template <int S>
int launch_sequence(const float *post, int32_t *states, const uint8_t *moves, float *qual_data,
                    float *base_probs, float *total_probs, char *sequence, char *qstring, int T, int N,
                    const ofk_phred_table_t &phred, hipStream_t st) {
    const size_t lds = (size_t)T * (4 + 4 + 1 + 1) + (size_t)(T + 1) * 4;
    if (lds > 64 * 1024) {  // beyond the default limit of dynamic LDS; the compute unit has 160 KB
        const hipError_t rc = hipFuncSetAttribute(reinterpret_cast<const void *>(&sequence_kernel<S>),
                                                  hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (rc != hipSuccess) return (int)rc;
    }
    hipLaunchKernelGGL((sequence_kernel<S>), dim3(N), dim3(kThreads), lds, st, post, states, moves, qual_data,
                       base_probs, total_probs, sequence, qstring, T, phred);
    return (int)hipGetLastError();
}

}  // namespace

extern "C" int ofk_sequence(const float *post, int32_t *states, const uint8_t *moves, float *qual_data,
                            float *base_probs, float *total_probs, char *sequence, char *qstring, int T, int N,
                            int state_len, const ofk_phred_table_t *phred, void *stream) {
    // the per-chunk tables live in LDS: 14 bytes per time step
    if (!post || !states || !moves || !qual_data || !base_probs || !total_probs || !sequence || !qstring ||
        !phred || T < 1 || T > OFK_MAX_T || N < 1)
        return OFK_BAD_ARGS;
    if (reinterpret_cast<uintptr_t>(qual_data) & 15u) return OFK_BAD_ARGS;
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (state_len) {
        case 3: return launch_sequence<64>(post, states, moves, qual_data, base_probs, total_probs, sequence, qstring, T, N, *phred, st);
        case 4: return launch_sequence<256>(post, states, moves, qual_data, base_probs, total_probs, sequence, qstring, T, N, *phred, st);
        case 5: return launch_sequence<1024>(post, states, moves, qual_data, base_probs, total_probs, sequence, qstring, T, N, *phred, st);
        default: return OFK_BAD_ARGS;
    }
}
