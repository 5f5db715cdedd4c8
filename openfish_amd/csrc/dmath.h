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

#include <math.h>
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

// Coefficients of e^r for |r| <= ln2/2, highest degree first: the degree-10 polynomial of least
// maximal relative error on that interval (2^-52.07 before rounding; found with the Remez exchange
// in 60-digit arithmetic); the constant term, exactly 1 so that e^0 = 1 exactly, is not in the
// list.  Then 1.5 * 2^52 (adding it rounds to an integer), log2(e) and -ln 2.
// A kernel passes the list as an argument, which keeps it in scalar registers; written as
// literals the compiler copies the values into vector registers at every use.
#define OFA_EXP_COEFS                                                                                    \
    {0x1.2727a6f878ec2p-22, 0x1.72f9854873e44p-19, 0x1.a01b6ce553964p-16, 0x1.a0197a4e972fcp-13,         \
     0x1.6c16c0c0ac0c6p-10, 0x1.1111112d49797p-7,  0x1.55555555933c6p-5,  0x1.555555554bc09p-3,          \
     0x1.ffffffffffe17p-2,  0x1.000000000001dp+0,  6755399441055744.0,    1.4426950408889634074,         \
     -0.69314718055994530942}
#define OFA_EXP_COEF_COUNT 13
OFA_HD double exp_reduced(double r, const double *c) {
    double p = c[0];
    p = __builtin_fma(p, r, c[1]);
    p = __builtin_fma(p, r, c[2]);
    p = __builtin_fma(p, r, c[3]);
    p = __builtin_fma(p, r, c[4]);
    p = __builtin_fma(p, r, c[5]);
    p = __builtin_fma(p, r, c[6]);
    p = __builtin_fma(p, r, c[7]);
    p = __builtin_fma(p, r, c[8]);
    p = __builtin_fma(p, r, c[9]);
    return __builtin_fma(p, r, 1.0);
}

// e^x for a double x (|x| < 1e9: the integer part of x*log2(e) is read from 32 bits); the scans
// call it with x = a float d <= 0.
// One-step argument reduction r = x - n ln2 with ln2 rounded to double: its error, |n| 2^-54
// relative to e^x, is |n| 2^(-54-|n|/0.69..) relative to 1, and the sums these exponentials
// enter are at least 1 (one term of every sum is e^0).  The scaling by 2^n is a true ldexp,
// which underflows to zero by itself.
OFA_HD double exp_ldexp(double x, const double *c) {
    const double t = __builtin_fma(x, c[11], c[10]);
    const double n = t - c[10];
    const double r = __builtin_fma(n, c[12], x);  // |r| <= ln2/2 (+ 1e-14)
    const double p = exp_reduced(r, c);
    return __builtin_ldexp(p, (int)(uint32_t)bits_of(t));
}
OFA_HD double exp_nonpos_ldexp(float d, const double *c) { return exp_ldexp((double)d, c); }

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

// The same logarithm with the table cell (and the power of two) taken from an approximation
// `near` of s, |near / s - 1| < 2^-18, so that the cell can be fetched before s is known: with k the
// exponent of `near` and c its cell, ln s = k ln2 + ln c + log1p(s 2^-k / c - 1), and the argument of
// log1p stays within 1/64 + 2^-17 in magnitude whichever side of a cell (or binade) boundary s itself
// falls on: the ninth power, the first one the series drops, stays below 2^-56.
OFA_HD LogCell log_cell_near(float near, const LogCell *table) { return table[(bits_of(near) >> 18) & 31u]; }
OFA_HD double log_1to5_with_cell(float s, float near, LogCell c, const double *series) {
    const int k = (int)(bits_of(near) >> 23) - 127;
    const double u = __builtin_ldexp((double)s, -k);
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

// RN32(m + ln s) as the CPU path forms it: the sum in double, one rounding.  ln 1 is exactly 0 on
// the CPU path; the table logarithm returns about 1e-18 there, which would show in a result whose
// m is zero.
OFA_HD float add_log_rounded(float m, float s, const LogCell *table, const double *series) {
    const float r = (float)((double)m + log_1to5_tab(s, table, series));
    return s == 1.0f ? m : r;
}

// max + ln(sum_i e^(v_i - max)) with the CPU path's roundings (reference src/decode_cpu.c:45-49):
// fp32 differences, the running sum rounded to fp32 after every term, one rounding of the final sum.
OFA_HD float lse5_cpu_rounding_tab(float v0, float v1, float v2, float v3, float v4, float m,
                                   const LogCell *table, const double *series, const double *ec) {
    float s = (float)exp_nonpos_ldexp(v0 - m, ec);
    s = (float)((double)s + exp_nonpos_ldexp(v1 - m, ec));
    s = (float)((double)s + exp_nonpos_ldexp(v2 - m, ec));
    s = (float)((double)s + exp_nonpos_ldexp(v3 - m, ec));
    s = (float)((double)s + exp_nonpos_ldexp(v4 - m, ec));
    return add_log_rounded(m, s, table, series);
}


// ---------------------------------------------------------------------------------------------
// Two-tier evaluation.  lse5_estimate computes the same quantity with the fp32 hardware
// exponential and logarithm and decides whether its rounded result is certain to be the fp32
// number the CPU path (reference src/decode_cpu.c:45-49) produces.  Where it is not certain
// ("unsettled"), the caller evaluates lse5_cpu_rounding_tab instead.
//
// With d_i = v_i - m (fp32, as on the CPU path) the CPU path's result is RN32(m + ln s_cpu),
// s_cpu the fp32 running sum of the double exponentials.  The estimate forms
//   t_i = RN32(d_i * c),  E_i = exp2(t_i),  s~ = fp32 running sum of E_i,  l2 = log2(s~),
//   r~ = RN32(m + l2 * ln2f)          (one fused multiply-add)
// and x~ = m + l2 * ln2f differs from x = m + ln s_cpu by at most eps.  With s~ in
// [2^k, 2^(k+1)) and all terms in units of 2^-24 = 5.96e-8:
//   8.5 * 2^k / s   roundings of the two running sums.  s_cpu against the exact sum S of the
//         e^{d_i}: the first term rounded to fp32 (half an ulp of a number <= 1: 0.5 absolute)
//         and four additions, each off by at most half an ulp of a partial sum <= s, i.e. by 2^k
//         absolute; s~ against the exact sum of the E_i: four fp32 additions, 2^k each.
//         Relative to s that is (0.5 + 8 * 2^k) / s <= 8.5 * 2^k / s
//   1.43 (S-1)/S   v_exp_f32: largest relative error found over every input in [-160, 0] is
//         1.423 * 2^-24; the term with d = 0 is exactly 1; (S-1)/S <= 0.5, 0.75, 0.8 for k = 0, 1, 2
//   0.88  argument of exp2: t_i = d_i c (1 + p), |p| <= 2^-24 + 1.34e-8 (c rounded to fp32), a
//         relative error |d_i| p of E_i; sum_i |d_i| e^{d_i} / S <= 0.718
//   0.70 * 2^k  v_log_f32: largest absolute error found over every input in [1, 5.01] is
//         1.0, 2.0, 4.0 * 2^-24 for s~ in [1,2), [2,4), [4,5.01]; times ln 2
//   0.12  ln2f against ln 2 (1.9e-9 * l2), rounding of the residual below, second-order terms
// The last four add up to 2.415, 3.463, 4.914 for k = 0, 1, 2, all at most 1.38 + 1.045 * 2^k.
// With mu = s~ / 2^(k+1) in [0.5, 1), 2^k / s = 1 / (2 mu) <= 1.5 - mu (the chord of a convex
// function), so that
//   eps = 14.13 - 8.5 mu + 1.045 * 2^k    (11.0 at s~ = 1, 6.7 just below 2, 12.0 at 2, ...)
// is a bound, evaluated from the bits of s~ with two fused multiply-adds; the constants below
// add 3 %.  The four hardware figures (1.43 for v_exp_f32; 1.0, 2.0, 4.0 for v_log_f32) and the
// identities exp2(0) = 1, log2(1) = 0 are premises about the device: tests/test_gpu_hw_math.py
// measures them over every fp32 input of those ranges on the device it runs on (probe.hip) and
// fails if one is exceeded.  The binade is read from s~ raised by 16 ulps: should s_cpu, within a dozen ulps
// of s~, reach the next binade, where half an ulp is twice as large, s~ counts as being there too.
//
// r~ is settled when no rounding boundary lies within eps of x~: with rho = x~ - r~ (exact up
// to one rounding: r~ - m is exact by Sterbenz' lemma once |m| >= 3.3, and smaller |m| are
// never settled because half an ulp of r~ is then below eps) and h = half an ulp of r~, the
// distance from x~ to the nearer boundary is at least h - |rho|.  A power of two has its lower
// boundary only a quarter of its ulp away: h is read from the exponent of the next smaller
// float, which is the binade below exactly for powers of two, so that one comparison serves
// every case.  Values below 2^-102 (zero included) come out with h <= 0 and are never settled.
// ---------------------------------------------------------------------------------------------
OFA_HD float exp2_hw(float x) {
#if defined(__HIP_DEVICE_COMPILE__)
    return __builtin_amdgcn_exp2f(x);
#else
    return exp2f(x);
#endif
}
OFA_HD float log2_hw(float x) {
#if defined(__HIP_DEVICE_COMPILE__)
    return __builtin_amdgcn_logf(x);
#else
    return log2f(x);
#endif
}

struct Lse5Estimate {
    float value;
    float sum;  // the fp32 estimate of the sum of exponentials, within 1e-6 (relative) of the CPU path's
    bool settled;
};
OFA_HD Lse5Estimate lse5_estimate(float v0, float v1, float v2, float v3, float v4, float m) {
    const float kLog2e = 1.44269504088896340736f, kLn2 = 0.69314718055994530942f;
    float s = exp2_hw((v0 - m) * kLog2e);
    s += exp2_hw((v1 - m) * kLog2e);
    s += exp2_hw((v2 - m) * kLog2e);
    s += exp2_hw((v3 - m) * kLog2e);
    s += exp2_hw((v4 - m) * kLog2e);
    const float kEps0 = 8.68e-7f, kEpsMu = 5.21e-7f, kEps1 = 6.42e-8f;
    const float l2 = log2_hw(s);
    Lse5Estimate e;
    e.sum = s;
    e.value = __builtin_fmaf(l2, kLn2, m);
    const float rho = __builtin_fmaf(l2, kLn2, -(e.value - m));
    const uint32_t rb = bits_of(e.value);
    // exponent field of the float below |r~|, lowered by 24; where that wraps, the sign bit survives the mask
    const float h = float_of(((rb & 0x7fffffffu) - ((24u << 23) + 1u)) & 0xff800000u);
    const uint32_t sb = bits_of(s) + 16u;
    const float mu = float_of((sb & 0x007fffffu) | 0x3f000000u);
    const float eps = __builtin_fmaf(mu, -kEpsMu, __builtin_fmaf(float_of(sb & 0x7f800000u), kEps1, kEps0));
    e.settled = h - __builtin_fabsf(rho) > eps;
    return e;
}

// the scan update in two tiers: the estimate where it is settled, the CPU roundings elsewhere
OFA_HD float lse5_two_tier(float v0, float v1, float v2, float v3, float v4, float m, const LogCell *table,
                           const double *series, const double *ec) {
    const Lse5Estimate e = lse5_estimate(v0, v1, v2, v3, v4, m);
    if (e.settled) return e.value;
    return lse5_cpu_rounding_tab(v0, v1, v2, v3, v4, m, table, series, ec);
}

}  // namespace ofa

#endif
