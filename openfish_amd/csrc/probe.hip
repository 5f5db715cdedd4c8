// Exhaustive error measurement of the two hardware transcendentals the scans and the beam
// search's merges rely on: v_exp_f32 over every fp32 in [-160, 0] and v_log_f32 over every fp32
// in [1, 5.01], against double arithmetic.  The two-tier evaluations (dmath.h lse5_estimate,
// beam.hip log_sum_exp_estimate) are exact only while these errors stay within the bounds their
// derivations budget; the GPU tests call this probe and assert those bounds on the device at hand.
#include <hip/hip_runtime.h>

#include "kernels.h"

namespace {

struct ProbeResult {
    unsigned long long exp_rel_max;     // bit patterns of non-negative doubles: ordered like the values
    unsigned long long log_abs_max[3];  // s in [1,2), [2,4), [4,5.01]
    unsigned int identities;            // bit 0: exp2(0) == 1, bit 1: exp2(-0) == 1, bit 2: log2(1) == 0, bit 3: log2(2) == 1
};

__global__ __launch_bounds__(256) void probe_exp_kernel(unsigned lo_bits, unsigned count, ProbeResult *res) {
    double worst = 0.0;
    for (unsigned i = blockIdx.x * blockDim.x + threadIdx.x; i < count; i += gridDim.x * blockDim.x) {
        const float t = __uint_as_float(lo_bits + i);  // negative floats: larger bit pattern = more negative
        const float e = __builtin_amdgcn_exp2f(t);
        const double exact = exp2((double)t);
        if (exact < 1.1754943508222875e-38) continue;  // below the normal range the result is flushed; its absolute error is negligible
        const double rel = fabs((double)e - exact) / exact;
        worst = rel > worst ? rel : worst;
    }
    atomicMax(&res->exp_rel_max, (unsigned long long)__double_as_longlong(worst));
}

__global__ __launch_bounds__(256) void probe_log_kernel(unsigned lo_bits, unsigned count, ProbeResult *res) {
    double worst[3] = {0.0, 0.0, 0.0};
    for (unsigned i = blockIdx.x * blockDim.x + threadIdx.x; i < count; i += gridDim.x * blockDim.x) {
        const float s = __uint_as_float(lo_bits + i);
        const float l = __builtin_amdgcn_logf(s);
        const double err = fabs((double)l - log2((double)s));
        const int c = s < 2.0f ? 0 : (s < 4.0f ? 1 : 2);
        worst[c] = err > worst[c] ? err : worst[c];
    }
    for (int c = 0; c < 3; ++c) atomicMax(&res->log_abs_max[c], (unsigned long long)__double_as_longlong(worst[c]));
}

__global__ void probe_identities_kernel(ProbeResult *res) {
    res->identities = (__builtin_amdgcn_exp2f(0.0f) == 1.0f ? 1u : 0u) | (__builtin_amdgcn_exp2f(-0.0f) == 1.0f ? 2u : 0u) |
                      (__builtin_amdgcn_logf(1.0f) == 0.0f ? 4u : 0u) | (__builtin_amdgcn_logf(2.0f) == 1.0f ? 8u : 0u);
}

}  // namespace

extern "C" int ofk_probe_hw_math(void *scratch32, void *stream) {
    if (!scratch32 || (reinterpret_cast<uintptr_t>(scratch32) & 7u)) return OFK_BAD_ARGS;
    hipStream_t st = static_cast<hipStream_t>(stream);
    ProbeResult *res = static_cast<ProbeResult *>(scratch32);
    static_assert(sizeof(ProbeResult) <= 40, "the caller provides 40 bytes");
    hipError_t e = hipMemsetAsync(res, 0, sizeof(ProbeResult), st);
    if (e != hipSuccess) return (int)e;
    const unsigned exp_lo = 0x80000000u, exp_hi = 0xC3200000u;  // -0.0f .. -160.0f
    const unsigned log_lo = 0x3F800000u, log_hi = 0x40A051ECu;  // 1.0f .. 5.01f
    hipLaunchKernelGGL(probe_exp_kernel, dim3(4096), dim3(256), 0, st, exp_lo, exp_hi - exp_lo + 1u, res);
    hipLaunchKernelGGL(probe_log_kernel, dim3(4096), dim3(256), 0, st, log_lo, log_hi - log_lo + 1u, res);
    hipLaunchKernelGGL(probe_identities_kernel, dim3(1), dim3(1), 0, st, res);
    return (int)hipGetLastError();
}
