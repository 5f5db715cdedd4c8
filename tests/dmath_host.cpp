// Host build of openfish_amd/csrc/dmath.h for the accuracy tests (tests/test_dmath.py).
#include <math.h>

#include "dmath.h"

static const double kSeries[6] = OFA_LOG_SERIES;
static const double kExp[OFA_EXP_COEF_COUNT] = OFA_EXP_COEFS;

extern "C" {

// largest error of exp_nonpos_ldexp against expl over the given floats: relative to the exact
// value if relative != 0, absolute otherwise
double max_err_exp(const float *d, long n, int relative) {
    double worst = 0;
    for (long i = 0; i < n; ++i) {
        const long double want = expl((long double)d[i]);
        const long double got = ofa::exp_nonpos_ldexp(d[i], kExp);
        const long double diff = fabsl(got - want);
        const double err = (double)((relative && want != 0) ? diff / want : diff);
        if (err > worst) worst = err;
    }
    return worst;
}

// largest absolute error of the table-driven logarithm against logl
double max_abs_err_log_tab(const float *s, long n) {
    ofa::LogCell table[32];
    for (int i = 0; i < 32; ++i) table[i] = ofa::log_cell(i);
    double worst = 0;
    for (long i = 0; i < n; ++i) {
        const double err = (double)fabsl((long double)ofa::log_1to5_tab(s[i], table, kSeries) - logl((long double)s[i]));
        if (err > worst) worst = err;
    }
    return worst;
}

// largest absolute error of the logarithm whose table cell comes from a neighbour `near` of s
// (s moved by up to `ulps` fp32 steps either way), against logl
double max_abs_err_log_near(const float *s, long n, int ulps) {
    ofa::LogCell table[32];
    for (int i = 0; i < 32; ++i) table[i] = ofa::log_cell(i);
    double worst = 0;
    for (long i = 0; i < n; ++i) {
        for (int d = -ulps; d <= ulps; d += (ulps > 0 ? ulps : 1)) {
            const float near = ofa::float_of(ofa::bits_of(s[i]) + (uint32_t)d);
            if (!(near >= 1.0f)) continue;
            const double got = ofa::log_1to5_with_cell(s[i], near, ofa::log_cell_near(near, table), kSeries);
            const double err = (double)fabsl((long double)got - logl((long double)s[i]));
            if (err > worst) worst = err;
        }
    }
    return worst;
}

// the CPU path's own arithmetic (libm exp/log in double, fp32 running sum)
static float lse5_libm(const float v[5], float m) {
    float acc = 0.0f;
    for (int i = 0; i < 5; ++i) acc = (float)((double)acc + exp((double)(v[i] - m)));
    return (float)((double)m + log((double)acc));
}

// number of 5-tuples on which lse5_cpu_rounding_tab differs from the libm version in any bit
long lse5_mismatches(const float *v, long n) {
    ofa::LogCell table[32];
    for (int i = 0; i < 32; ++i) table[i] = ofa::log_cell(i);
    long bad = 0;
    for (long i = 0; i < n; ++i) {
        const float *p = v + 5 * i;
        float m = p[0];
        for (int k = 1; k < 5; ++k) m = m > p[k] ? m : p[k];
        const float a = ofa::lse5_cpu_rounding_tab(p[0], p[1], p[2], p[3], p[4], m, table, kSeries, kExp);
        const float b = lse5_libm(p, m);
        if (memcmp(&a, &b, 4) != 0) ++bad;
    }
    return bad;
}

// two-tier update against the libm version: returns the number of 5-tuples whose estimate was
// taken as settled although it differs from the libm result (must be zero), stores the number of
// unsettled estimates and the number of results of the whole two-tier update that differ
long two_tier_wrongly_settled(const float *v, long n, long *unsettled, long *mismatches) {
    ofa::LogCell table[32];
    for (int i = 0; i < 32; ++i) table[i] = ofa::log_cell(i);
    long wrong = 0, open = 0, bad = 0;
    for (long i = 0; i < n; ++i) {
        const float *p = v + 5 * i;
        float m = p[0];
        for (int k = 1; k < 5; ++k) m = m > p[k] ? m : p[k];
        const float want = lse5_libm(p, m);
        const ofa::Lse5Estimate e = ofa::lse5_estimate(p[0], p[1], p[2], p[3], p[4], m);
        if (!e.settled) ++open;
        else if (memcmp(&e.value, &want, 4) != 0) ++wrong;
        const float got = ofa::lse5_two_tier(p[0], p[1], p[2], p[3], p[4], m, table, kSeries, kExp);
        if (memcmp(&got, &want, 4) != 0) ++bad;
    }
    *unsettled = open;
    *mismatches = bad;
    return wrong;
}
}
