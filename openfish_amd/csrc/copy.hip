// A plain device-to-device copy kernel of known traffic (bytes read = bytes written =
// the size given).  It exists for measurement: hardware counters of the decode
// kernels are scaled by what the same counters report for this kernel.
#include <hip/hip_runtime.h>

#include "kernels.h"

namespace {

typedef uint32_t Vec16 __attribute__((ext_vector_type(4)));

// streaming loads and stores: nothing is read twice, nothing needs to stay in a cache
__global__ __launch_bounds__(256) void copy_kernel(const Vec16 *__restrict__ src, Vec16 *__restrict__ dst, size_t n16) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += stride)
        __builtin_nontemporal_store(__builtin_nontemporal_load(&src[i]), &dst[i]);
}

}  // namespace

extern "C" int ofk_copy(void *dst, const void *src, size_t bytes, void *stream) {
    if (!dst || !src || (bytes & 15u) || ((reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(src)) & 15u))
        return OFK_BAD_ARGS;
    if (bytes == 0) return 0;
    const size_t n16 = bytes / 16;
    size_t blocks = (n16 + 255) / 256;
    if (blocks > 256 * 64) blocks = 256 * 64;  // 64 workgroups per compute unit (measured best), grid-stride beyond
    hipLaunchKernelGGL(copy_kernel, dim3((unsigned)blocks), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<const Vec16 *>(src), static_cast<Vec16 *>(dst), n16);
    return (int)hipGetLastError();
}
