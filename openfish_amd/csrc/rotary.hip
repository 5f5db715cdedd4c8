// In-place rotary embedding on half data with fp32 sin/cos tables, gfx950.
//
// For every (batch, seq, head, rot < rotary_half) the pair
//   x0 = x[batch*stride_batch + seq*stride_seq + head*stride_head + rot], x1 = x0's partner at +rotary_half
// becomes (x0*cos - x1*sin, x0*sin + x1*cos) with cos/sin taken at [seq][rot]
// (reference src/rotary_emb_hip.h:36-70, CPU twin src/nn_cpu.c:10-39).  Products and
// sums are separate fp32 operations (no fused multiply-add), the result is rounded
// to half once.  The op is pure streaming: the fast path moves 8 pairs per thread
// with 128-bit loads and stores; a scalar path covers shapes that are not
// multiples of 8.
#include <hip/hip_runtime.h>

#include "kernels.h"

namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float float4v __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(256) void rotary_vec8_kernel(_Float16 *__restrict__ x, const float *__restrict__ sin_buf,
                                                          const float *__restrict__ cos_buf, long total, int seqlen,
                                                          int nheads, int groups, int rotary_half, long stride_batch,
                                                          long stride_seq, long stride_head) {
    const long id = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (id >= total) return;
    const int grp = (int)(id % groups);
    long rest = id / groups;
    const int head = (int)(rest % nheads);
    rest /= nheads;
    const int seq = (int)(rest % seqlen);
    const long batch = rest / seqlen;
    const int rot = grp * 8;

    _Float16 *p0 = x + batch * stride_batch + (long)seq * stride_seq + (long)head * stride_head + rot;
    _Float16 *p1 = p0 + rotary_half;
    const long tab = (long)seq * rotary_half + rot;
    const float4v c0 = *reinterpret_cast<const float4v *>(cos_buf + tab);
    const float4v c1 = *reinterpret_cast<const float4v *>(cos_buf + tab + 4);
    const float4v s0 = *reinterpret_cast<const float4v *>(sin_buf + tab);
    const float4v s1 = *reinterpret_cast<const float4v *>(sin_buf + tab + 4);
    const half8 a = *reinterpret_cast<const half8 *>(p0);
    const half8 b = *reinterpret_cast<const half8 *>(p1);
    half8 ra, rb;
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        const float c = k < 4 ? c0[k & 3] : c1[k & 3];
        const float s = k < 4 ? s0[k & 3] : s1[k & 3];
        const float x0 = (float)a[k], x1 = (float)b[k];
        ra[k] = (_Float16)(x0 * c - x1 * s);
        rb[k] = (_Float16)(x0 * s + x1 * c);
    }
    *reinterpret_cast<half8 *>(p0) = ra;
    *reinterpret_cast<half8 *>(p1) = rb;
}

__global__ __launch_bounds__(256) void rotary_scalar_kernel(_Float16 *__restrict__ x, const float *__restrict__ sin_buf,
                                                            const float *__restrict__ cos_buf, long total, int seqlen,
                                                            int nheads, int rotary_half, long stride_batch,
                                                            long stride_seq, long stride_head) {
    const long id = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (id >= total) return;
    const int rot = (int)(id % rotary_half);
    long rest = id / rotary_half;
    const int head = (int)(rest % nheads);
    rest /= nheads;
    const int seq = (int)(rest % seqlen);
    const long batch = rest / seqlen;
    _Float16 *p0 = x + batch * stride_batch + (long)seq * stride_seq + (long)head * stride_head + rot;
    _Float16 *p1 = p0 + rotary_half;
    const float c = cos_buf[(long)seq * rotary_half + rot];
    const float s = sin_buf[(long)seq * rotary_half + rot];
    const float x0 = (float)*p0, x1 = (float)*p1;
    *p0 = (_Float16)(x0 * c - x1 * s);
    *p1 = (_Float16)(x0 * s + x1 * c);
}

}  // namespace

extern "C" int ofk_rotary_emb(void *x, const float *sin_buf, const float *cos_buf, int batch, int seqlen,
                              int nheads, int rotary_half, long stride_batch, long stride_seq,
                              long stride_head, void *stream) {
    if (!x || !sin_buf || !cos_buf || batch < 0 || seqlen < 0 || nheads < 0 || rotary_half < 0) return OFK_BAD_ARGS;
    if (batch == 0 || seqlen == 0 || nheads == 0 || rotary_half == 0) return 0;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const bool vec = rotary_half % 8 == 0 && stride_batch % 8 == 0 && stride_seq % 8 == 0 && stride_head % 8 == 0 &&
                     ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(sin_buf) |
                       reinterpret_cast<uintptr_t>(cos_buf)) & 15u) == 0;
    if (vec) {
        const int groups = rotary_half / 8;
        const long total = (long)batch * seqlen * nheads * groups;
        const long blocks = (total + 255) / 256;
        if (blocks > 0x7fffffffL) return OFK_BAD_ARGS;
        hipLaunchKernelGGL(rotary_vec8_kernel, dim3((unsigned)blocks), dim3(256), 0, st, static_cast<_Float16 *>(x),
                           sin_buf, cos_buf, total, seqlen, nheads, groups, rotary_half, stride_batch, stride_seq,
                           stride_head);
    } else {
        const long total = (long)batch * seqlen * nheads * rotary_half;
        const long blocks = (total + 255) / 256;
        if (blocks > 0x7fffffffL) return OFK_BAD_ARGS;
        hipLaunchKernelGGL(rotary_scalar_kernel, dim3((unsigned)blocks), dim3(256), 0, st, static_cast<_Float16 *>(x),
                           sin_buf, cos_buf, total, seqlen, nheads, rotary_half, stride_batch, stride_seq,
                           stride_head);
    }
    return (int)hipGetLastError();
}
