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

// [rows][S][5] fp16 with a leading blank/stay column -> [rows][S][4]: the four step columns
__global__ __launch_bounds__(256) void drop_blank_kernel(const uint16_t *__restrict__ src, uint2 *__restrict__ dst,
                                                         size_t groups) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t g = (size_t)blockIdx.x * blockDim.x + threadIdx.x; g < groups; g += stride) {
        const uint16_t *p = src + g * 5;
        uint2 v;
        v.x = (uint32_t)p[1] | ((uint32_t)p[2] << 16);
        v.y = (uint32_t)p[3] | ((uint32_t)p[4] << 16);
        dst[g] = v;
    }
}

}  // namespace

extern "C" int ofk_drop_blank_column(const void *scores5, void *scores4, size_t groups, void *stream) {
    if (!scores5 || !scores4 || (reinterpret_cast<uintptr_t>(scores4) & 7u) || (reinterpret_cast<uintptr_t>(scores5) & 1u))
        return OFK_BAD_ARGS;
    if (groups == 0) return 0;
    size_t blocks = (groups + 255) / 256;
    if (blocks > 256 * 32) blocks = 256 * 32;
    hipLaunchKernelGGL(drop_blank_kernel, dim3((unsigned)blocks), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<const uint16_t *>(scores5), static_cast<uint2 *>(scores4), groups);
    return (int)hipGetLastError();
}

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
