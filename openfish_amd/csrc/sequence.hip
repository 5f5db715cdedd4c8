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
    char *__restrict__ sequence, char *__restrict__ qstring, int T, ofk_phred_table_t phred,
    const float *__restrict__ path_sums) {
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
        float prob;
        if (path_sums) {  // the sum below, taken for every state by path_sums_kernel: one read instead of nine
            prob = path_sums[((size_t)n * T + t) * S + st];
        } else {
            const float *p = post_n + (size_t)(t + 1) * S;
            prob = p[st];
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


// ---------------------------------------------------------------------------------------------
// For every chunk, time step and state: the posterior of the k-mer plus that of its distinct
// one-base shifts, summed in the CPU path's order -- what step 1 of sequence_kernel gathers for
// the one state on the path.  Those nine scattered reads per time step fetch about half of the
// posteriors, 64 bytes for every 4 wanted, and made up most of that kernel's time; they come
// after the beam search, which leaves most of the machine idle for a millisecond.  This kernel
// runs beside the search, reads every row once, in order, and the sequence stage then takes one
// value per time step.
//
// A wave owns whole rows (four at a time with 64 states) and keeps the current one in LDS, 256
// floats per 64 lanes; lane j holds states 4j .. 4j+3 of each 256.  Those four share their
// four predecessors (st >> 2) + b * S/4, and the successors 4 * (st mod S/4) + b of a state are
// four neighbours in the row: eight LDS reads per lane cover all 32 values.  Which of a state's
// eight neighbours count (not the state itself, not an earlier neighbour) does not depend on
// the time step and is worked out once per lane.  A wave's LDS operations complete in order, so
// the waves of a group never wait for each other.
// ---------------------------------------------------------------------------------------------
template <int S>
__global__ __launch_bounds__(256) void path_sums_kernel(const float *__restrict__ post, float *__restrict__ sums,
                                                        int T, long rows) {
    constexpr int Q = S / 4;
    constexpr int G = S >= 256 ? S / 256 : 1;       // float4 pieces of a row per lane
    constexpr int kRowsPerTile = S >= 256 ? 1 : 4;  // rows a wave takes at a time
    constexpr int kTile = S >= 256 ? S : 256;       // floats
    __shared__ __attribute__((aligned(16))) float tiles[4][kTile];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    float *tile = tiles[wave];
    const int sub = S >= 256 ? 0 : lane >> 4;           // row of the tile this lane works on
    const int j0 = S >= 256 ? lane : lane & 15;         // quad of states within 256 (within the row, with 64 states)
    float *row = tile + (S >= 256 ? 0 : 64 * sub);      // this lane's row in LDS

    // per state: which neighbours are added (bit k: neighbour k, predecessors at even k)
    uint32_t fresh[G][4];
#pragma unroll
    for (int g = 0; g < G; ++g) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int st = 4 * (j0 + 64 * g) + i;
            int nb[8];
#pragma unroll
            for (int b = 0; b < 4; ++b) {
                nb[2 * b] = (st >> 2) + Q * b;
                nb[2 * b + 1] = ((st << 2) & (S - 1)) + b;
            }
            uint32_t bits = 0;
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                bool f = nb[k] != st;
#pragma unroll
                for (int m = 0; m < k; ++m) f = f && nb[m] != nb[k];
                bits |= f ? 1u << k : 0u;
            }
            fresh[g][i] = bits;
        }
    }

    const long tiles_n = (rows + kRowsPerTile - 1) / kRowsPerTile;
    const long step = (long)gridDim.x * 4;
    long tix = (long)blockIdx.x * 4 + wave;
    // row r of the output is time step r % T of chunk r / T and reads row r % T + 1 of that chunk's posteriors
    auto in_row = [&](long r) { return post + ((size_t)(r / T) * (size_t)(T + 1) + (size_t)(r % T) + 1) * S; };
    float4 cur[G], nxt[G];
    auto fetch = [&](long t_ix, float4 (&v)[G]) {
        const long r = t_ix * kRowsPerTile + sub;
#pragma unroll
        for (int g = 0; g < G; ++g)
            v[g] = (t_ix < tiles_n && r < rows) ? *reinterpret_cast<const float4 *>(in_row(r) + 4 * (j0 + 64 * g))
                                                : make_float4(0.f, 0.f, 0.f, 0.f);
    };
    fetch(tix, cur);
    for (; tix < tiles_n; tix += step) {
        fetch(tix + step, nxt);
#pragma unroll
        for (int g = 0; g < G; ++g) *reinterpret_cast<float4 *>(row + 4 * (j0 + 64 * g)) = cur[g];
        __builtin_amdgcn_wave_barrier();
        const long r = tix * kRowsPerTile + sub;
#pragma unroll
        for (int g = 0; g < G; ++g) {
            const int j = j0 + 64 * g;  // the lane's states 4j .. 4j+3 share their predecessors j + b * Q
            float prev[4];
#pragma unroll
            for (int b = 0; b < 4; ++b) prev[b] = row[j + Q * b];
            const float own[4] = {cur[g].x, cur[g].y, cur[g].z, cur[g].w};
            float out[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int st = 4 * j + i;
                const float4 nx = *reinterpret_cast<const float4 *>(row + 4 * (st & (Q - 1)));
                const float next[4] = {nx.x, nx.y, nx.z, nx.w};
                float prob = own[i];  // fp32 sums in the CPU path's order
#pragma unroll
                for (int b = 0; b < 4; ++b) {
                    const float with_prev = prob + prev[b];
                    prob = (fresh[g][i] >> (2 * b)) & 1u ? with_prev : prob;
                    const float with_next = prob + next[b];
                    prob = (fresh[g][i] >> (2 * b + 1)) & 1u ? with_next : prob;
                }
                out[i] = prob;
            }
            if (r < rows)
                *reinterpret_cast<float4 *>(sums + (size_t)r * S + 4 * j) = make_float4(out[0], out[1], out[2], out[3]);
        }
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int g = 0; g < G; ++g) cur[g] = nxt[g];
    }
}

template <int S>
int launch_path_sums(const float *post, float *sums, int T, int N, hipStream_t st) {
    const long rows = (long)N * T;
    // Half as many workgroups as chunks, up to one per compute unit (one wave per SIMD): with 512
    // chunks of 256 states the kernel then ends well inside the beam search it runs beside and does
    // not slow it (measured: 256 groups 1.185 ms of search against 1.183 alone, 512 groups 1.195,
    // 1024 groups 1.27; 128 groups outlast the search).
    int wgs = N / 2;
    wgs = wgs < 64 ? 64 : (wgs > 256 ? 256 : wgs);
    hipLaunchKernelGGL((path_sums_kernel<S>), dim3(wgs), dim3(256), 0, st, post, sums, T, rows);
    return (int)hipGetLastError();
}

template <int S>
int launch_sequence(const float *post, int32_t *states, const uint8_t *moves, float *qual_data,
                    float *base_probs, float *total_probs, char *sequence, char *qstring, int T, int N,
                    const ofk_phred_table_t &phred, const float *path_sums, hipStream_t st) {
    const size_t lds = (size_t)T * (4 + 4 + 1 + 1) + (size_t)(T + 1) * 4;
    if (lds > 64 * 1024) {  // beyond the default limit of dynamic LDS; the compute unit has 160 KB
        const hipError_t rc = hipFuncSetAttribute(reinterpret_cast<const void *>(&sequence_kernel<S>),
                                                  hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (rc != hipSuccess) return (int)rc;
    }
    hipLaunchKernelGGL((sequence_kernel<S>), dim3(N), dim3(kThreads), lds, st, post, states, moves, qual_data,
                       base_probs, total_probs, sequence, qstring, T, phred, path_sums);
    return (int)hipGetLastError();
}

}  // namespace

extern "C" int ofk_path_sums(const float *post, float *sums, int T, int N, int state_len, void *stream) {
    if (!post || !sums || T < 1 || N < 1) return OFK_BAD_ARGS;
    if ((reinterpret_cast<uintptr_t>(post) | reinterpret_cast<uintptr_t>(sums)) & 15u) return OFK_BAD_ARGS;
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (state_len) {
        case 3: return launch_path_sums<64>(post, sums, T, N, st);
        case 4: return launch_path_sums<256>(post, sums, T, N, st);
        case 5: return launch_path_sums<1024>(post, sums, T, N, st);
        default: return OFK_BAD_ARGS;
    }
}

extern "C" int ofk_sequence(const float *post, int32_t *states, const uint8_t *moves, float *qual_data,
                            float *base_probs, float *total_probs, char *sequence, char *qstring, int T, int N,
                            int state_len, const ofk_phred_table_t *phred, const float *path_sums, void *stream) {
    // the per-chunk tables live in LDS: 14 bytes per time step
    if ((!post && !path_sums) || !states || !moves || !qual_data || !base_probs || !total_probs || !sequence || !qstring ||
        !phred || T < 1 || T > OFK_MAX_T || N < 1)
        return OFK_BAD_ARGS;
    if (reinterpret_cast<uintptr_t>(qual_data) & 15u) return OFK_BAD_ARGS;
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (state_len) {
        case 3: return launch_sequence<64>(post, states, moves, qual_data, base_probs, total_probs, sequence, qstring, T, N, *phred, path_sums, st);
        case 4: return launch_sequence<256>(post, states, moves, qual_data, base_probs, total_probs, sequence, qstring, T, N, *phred, path_sums, st);
        case 5: return launch_sequence<1024>(post, states, moves, qual_data, base_probs, total_probs, sequence, qstring, T, N, *phred, path_sums, st);
        default: return OFK_BAD_ARGS;
    }
}
