// Host build of openfish_amd/csrc/dmath.h for the accuracy tests (tests/test_dmath.py).
#include <math.h>

#include "dmath.h"

extern "C" {

// largest relative error of exp_nonpos against expl over the given floats
double max_rel_err_exp(const float *d, long n) {
    double worst = 0;
    for (long i = 0; i < n; ++i) {
        const long double want = expl((long double)d[i]);
        const long double got = ofa::exp_nonpos(d[i]);
        const double rel = (double)fabsl((got - want) / want);
        if (rel > worst) worst = rel;
    }
    return worst;
}

double max_rel_err_log(const float *s, long n) {
    double worst = 0;
    for (long i = 0; i < n; ++i) {
        const long double want = logl((long double)s[i]);
        const long double got = ofa::log_1to5(s[i]);
        const double err = want == 0 ? (double)fabsl(got) : (double)fabsl((got - want) / want);
        if (err > worst) worst = err;
    }
    return worst;
}

// largest absolute error of log1p_exp_neg against log1pl(expl(-gap))
double max_abs_err_lse2(const float *gap, long n) {
    double worst = 0;
    for (long i = 0; i < n; ++i) {
        const long double want = log1pl(expl(-(long double)gap[i]));
        const double err = (double)fabsl((long double)ofa::log1p_exp_neg(gap[i]) - want);
        if (err > worst) worst = err;
    }
    return worst;
}

// log(e^x + e^y) as the CPU path computes it vs. with log1p_exp_neg: count of differing results
long lse2_mismatches(const float *xy, long n) {
    long bad = 0;
    for (long i = 0; i < n; ++i) {
        const float x = xy[2 * i], y = xy[2 * i + 1];
        const float gap = fabsf(x - y), top = x > y ? x : y;
        const float a = (float)((double)top + (gap < 17.0f ? log(1.0 + exp(-(double)gap)) : 0.0));
        const float b = (float)((double)top + (gap < 17.0f ? ofa::log1p_exp_neg(gap) : 0.0));
        if (memcmp(&a, &b, 4) != 0) ++bad;
    }
    return bad;
}

double max_rel_err_exp_ldexp(const float *d, long n) {
    double worst = 0;
    for (long i = 0; i < n; ++i) {
        const long double want = expl((long double)d[i]);
        const long double got = ofa::exp_nonpos_ldexp(d[i]);
        const double rel = want == 0 ? (double)fabsl(got) : (double)fabsl((got - want) / want);
        if (rel > worst) worst = rel;
    }
    return worst;
}

double max_abs_err_log_tab(const float *s, long n) {
    ofa::LogCell table[32];
    for (int i = 0; i < 32; ++i) table[i] = ofa::log_cell(i);
    double worst = 0;
    for (long i = 0; i < n; ++i) {
        const double err = (double)fabsl((long double)ofa::log_1to5_tab(s[i], table) - logl((long double)s[i]));
        if (err > worst) worst = err;
    }
    return worst;
}

// the CPU path's own arithmetic (libm exp/log in double, fp32 running sum)
static float lse5_libm(const float v[5], float m) {
    float acc = 0.0f;
    for (int i = 0; i < 5; ++i) acc = (float)((double)acc + exp((double)(v[i] - m)));
    return (float)((double)m + log((double)acc));
}

static ofa::LogCell g_table[32];
static int g_table_ready = 0;

// number of 5-tuples on which lse5_cpu_rounding differs from the libm version in any bit
long lse5_mismatches(const float *v, long n) {
    if (!g_table_ready) {
        for (int i = 0; i < 32; ++i) g_table[i] = ofa::log_cell(i);
        g_table_ready = 1;
    }
    long bad = 0;
    for (long i = 0; i < n; ++i) {
        const float *p = v + 5 * i;
        float m = p[0];
        for (int k = 1; k < 5; ++k) m = m > p[k] ? m : p[k];
        const float a = ofa::lse5_cpu_rounding(p[0], p[1], p[2], p[3], p[4], m);
        const float b = lse5_libm(p, m);
        if (memcmp(&a, &b, 4) != 0) ++bad;
        const float c = ofa::lse5_cpu_rounding_tab(p[0], p[1], p[2], p[3], p[4], m, g_table);
        if (memcmp(&c, &b, 4) != 0) ++bad;
    }
    return bad;
}
}
