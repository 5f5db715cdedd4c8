// Double-precision exp and log for the scans, written for the narrow domains the
// scans need so that they cost a few dozen full-rate fp64 FMAs instead of a
// general libm call:
//   exp_nonpos_ldexp(d) : e^d for a float d <= 0, absolute error below 2^-51
//                         (relative error below 2^-50 for d >= -5.5)
//   log_1to5_tab(s)     : ln(s) for a float s in [1, 5] (a sum of five terms <= 1, one of
//                         which is exactly 1) from a 32-entry table of (1/c, ln c),
//                         absolute error below 2^-51
// The CPU path evaluates exp and log in double and then rounds to fp32 (reference
// src/decode_cpu.c:45-49); these stand in for its libm calls.  With the errors above
// a result can round to a different fp32 value only when the exact value lies
// within 2^-50 (relative) of a rounding boundary.
//
// The functions compile for host and device; the host build is what the accuracy
// test links.
#ifndef OPENFISH_AMD_DMATH_H
#define OPENFISH_AMD_DMATH_H

#include <stdint.h>
#include <string.h>

#if defined(__HIPCC__)
#define OFA_HD __host__ __device__ __forceinline__
#else
#define OFA_HD static inline
#endif

namespace ofa {

OFA_HD uint64_t bits_of(double x) {
    uint64_t u;
    memcpy(&u, &x, sizeof u);
    return u;
}
OFA_HD double double_of(uint64_t u) {
    double x;
    memcpy(&x, &u, sizeof x);
    return x;
}
OFA_HD uint32_t bits_of(float x) {
    uint32_t u;
    memcpy(&u, &x, sizeof u);
    return u;
}
OFA_HD float float_of(uint32_t u) {
    float x;
    memcpy(&x, &u, sizeof x);
    return x;
}

// e^r for |r| <= ln2/2: the degree-10 polynomial of least maximal relative error on that
// interval (2^-52.07 before rounding; found with the Remez exchange in 60-digit arithmetic).
// The constant term is exactly 1, so e^0 = 1 exactly.
OFA_HD double exp_reduced(double r) {
    double p = 0x1.2727a6f878ec2p-22;
    p = __builtin_fma(p, r, 0x1.72f9854873e44p-19);
    p = __builtin_fma(p, r, 0x1.a01b6ce553964p-16);
    p = __builtin_fma(p, r, 0x1.a0197a4e972fcp-13);
    p = __builtin_fma(p, r, 0x1.6c16c0c0ac0c6p-10);
    p = __builtin_fma(p, r, 0x1.1111112d49797p-7);
    p = __builtin_fma(p, r, 0x1.55555555933c6p-5);
    p = __builtin_fma(p, r, 0x1.555555554bc09p-3);
    p = __builtin_fma(p, r, 0x1.ffffffffffe17p-2);
    p = __builtin_fma(p, r, 0x1.000000000001dp+0);
    return __builtin_fma(p, r, 1.0);
}

// e^d for a float d <= 0 (|d| < 1e9: the integer part of d*log2(e) is read from 32 bits).
// One-step argument reduction r = d - n ln2 with ln2 rounded to double: its error, |n| 2^-54
// relative to e^d, is |n| 2^(-54-|n|/0.69..) relative to 1, and the sums these exponentials
// enter are at least 1 (one term of every sum is e^0).  The scaling by 2^n is a true ldexp,
// which underflows to zero by itself.
OFA_HD double exp_nonpos_ldexp(float d) {
    const double x = (double)d;
    const double kShift = 6755399441055744.0;  // 1.5 * 2^52: adding it rounds to an integer
    const double kLog2e = 1.4426950408889634074;
    const double kLn2 = 0.69314718055994530942;
    const double t = __builtin_fma(x, kLog2e, kShift);
    const double n = t - kShift;
    const double r = __builtin_fma(n, -kLn2, x);  // |r| <= ln2/2 (+ 1e-14)
    const double p = exp_reduced(r);
    return __builtin_ldexp(p, (int)(uint32_t)bits_of(t));
}

// k*ln2 + ln(1 + f) for f in [sqrt(1/2) - 1, sqrt(2) - 1]:
// ln(1 + f) = 2 atanh(z), z = f / (2 + f), |z| <= 0.1716.
OFA_HD double log_core(double f, int k) {
    const double den = 2.0 + f;
#if defined(__HIP_DEVICE_COMPILE__)
    double y = (double)__builtin_amdgcn_rcpf((float)den);
#else
    double y = (double)(1.0f / (float)den);
#endif
    y = __builtin_fma(__builtin_fma(-den, y, 1.0), y, y);  // Newton: 2^-22 -> 2^-44
    y = __builtin_fma(__builtin_fma(-den, y, 1.0), y, y);  // -> full double
    double z = f * y;
    z = __builtin_fma(__builtin_fma(-z, den, f), y, z);    // residual correction of the quotient
    const double w = z * z;  // <= 0.02944; the series is cut after w^9/21 < 2^-55
    double p = 1.0 / 19.0;
    p = __builtin_fma(p, w, 1.0 / 17.0);
    p = __builtin_fma(p, w, 1.0 / 15.0);
    p = __builtin_fma(p, w, 1.0 / 13.0);
    p = __builtin_fma(p, w, 1.0 / 11.0);
    p = __builtin_fma(p, w, 1.0 / 9.0);
    p = __builtin_fma(p, w, 1.0 / 7.0);
    p = __builtin_fma(p, w, 1.0 / 5.0);
    p = __builtin_fma(p, w, 1.0 / 3.0);
    const double z2 = z + z;
    const double lu = __builtin_fma(z2 * w, p, z2);
    const double kLn2 = 0.69314718055994530942;
    return __builtin_fma((double)k, kLn2, lu);
}

// Table-driven ln(s), s a float in [1, 5].  The mantissa interval [1, 2) is cut into 32
// cells with centres c_i = 1 + (2i + 1)/64; entry i holds inv = fl(1/c_i) and
// lnc = -ln(inv).  For s = 2^k * u:  ln(s) = k ln2 + lnc + log1p(u * inv - 1), and
// |u * inv - 1| <= 1/64 lets the series stop at the eighth power (next term < 2^-57).
struct LogCell {
    double inv, lnc;
};
OFA_HD LogCell log_cell(int i) {
    LogCell c;
    c.inv = 1.0 / (1.0 + (2 * i + 1) / 64.0);                 // in (0.5, 1)
    const bool low = c.inv < 0.70710678118654752;
    c.lnc = -log_core(low ? 2.0 * c.inv - 1.0 : c.inv - 1.0, low ? -1 : 0);  // differences exact
    return c;
}
// Coefficients -1/8, 1/7, ..., 1/3 of the series; the caller passes them from memory the scalar
// unit can read (on the device: constant memory), which keeps them in scalar registers for the
// whole kernel; written as literals they would be copied into vector registers at every use.
#define OFA_LOG_SERIES {-1.0 / 8.0, 1.0 / 7.0, -1.0 / 6.0, 1.0 / 5.0, -1.0 / 4.0, 1.0 / 3.0}
OFA_HD double log_1to5_tab(float s, const LogCell *table, const double *series) {
    const uint32_t b = bits_of(s);
    const int k = (int)(b >> 23) - 127;
    const LogCell c = table[(b >> 18) & 31u];
    const double u = (double)float_of((b & 0x007fffffu) | 0x3f800000u);
    const double r = __builtin_fma(u, c.inv, -1.0);
    double q = series[0];
    q = __builtin_fma(q, r, series[1]);
    q = __builtin_fma(q, r, series[2]);
    q = __builtin_fma(q, r, series[3]);
    q = __builtin_fma(q, r, series[4]);
    q = __builtin_fma(q, r, series[5]);
    q = __builtin_fma(q, r, -0.5);
    q = __builtin_fma(q, r, 1.0);
    const double lu = __builtin_fma(q, r, c.lnc);
    const double kLn2 = 0.69314718055994530942;
    return __builtin_fma((double)k, kLn2, lu);
}

// max + ln(sum_i e^(v_i - max)) with the CPU path's roundings (reference src/decode_cpu.c:45-49):
// fp32 differences, the running sum rounded to fp32 after every term, one rounding of the final sum.
OFA_HD float lse5_cpu_rounding_tab(float v0, float v1, float v2, float v3, float v4, float m,
                                   const LogCell *table, const double *series) {
    float s = (float)exp_nonpos_ldexp(v0 - m);
    s = (float)((double)s + exp_nonpos_ldexp(v1 - m));
    s = (float)((double)s + exp_nonpos_ldexp(v2 - m));
    s = (float)((double)s + exp_nonpos_ldexp(v3 - m));
    s = (float)((double)s + exp_nonpos_ldexp(v4 - m));
    return (float)((double)m + log_1to5_tab(s, table, series));
}

}  // namespace ofa

#endif
