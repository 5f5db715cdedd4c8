/*
 * Host side of the MI355X decoder: the public openfish entry points and the
 * stage-level C-ABI, in C, above the kernel launchers of kernels.h.
 *
 * One decode is   bwd scan -> { beam search || fwd+posterior scan } -> sequence   on two streams
 * (the beam search needs only scores and bwd, the posterior only feeds the quality stage, reference
 * src/beam_search.c:193,450) while the beam search leaves the machine idle, and   scans + posterior
 * (one kernel) -> { beam search || per-state sums of posteriors } -> sequence   for larger batches and
 * 1024 states; every call chooses unless the gpubuf says which (split_by_default).  The sequence stage
 * writes bases and qualities into pinned host memory itself.  Errors follow the reference convention
 * (reference src/hip_utils.h:11-28, src/error.h:44-72): message on stderr, then exit.
 */
#include <errno.h>
#include <float.h>
#include <math.h>
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <hip/hip_runtime_api.h>

#include <openfish/openfish.h>
#include <openfish/openfish_amd.h>
#include <openfish/openfish_error.h>

#include "kernels.h"

/* ---- logging (reference src/error.c:33-41) -------------------------------- */

static enum openfish_log_level_opt g_log_level = OPENFISH_LOG_VERB;

enum openfish_log_level_opt get_openfish_log_level(void) { return g_log_level; }
void set_openfish_log_level(enum openfish_log_level_opt level) { g_log_level = level; }

void openfish_log_emit(enum openfish_log_level_opt need, const char *tag, const char *colour,
                       const char *func, const char *file, int line, int where, const char *fmt, ...) {
    if (g_log_level < need) return;
    va_list ap;
    if (colour) fprintf(stderr, "[%s::%s]%s ", func, tag, colour);
    else fprintf(stderr, "[%s] %s: ", tag, func);
    va_start(ap, fmt);
    vfprintf(stderr, fmt, ap);
    va_end(ap);
    if (colour) fputs("\033[0m", stderr);
    if (where) fprintf(stderr, " At %s:%d", file, line);
    fputc('\n', stderr);
}

/* ---- error convention ------------------------------------------------------ */

#define HIP_OK(call)                                                                              \
    do {                                                                                          \
        hipError_t e_ = (call);                                                                   \
        if (e_ != hipSuccess) {                                                                   \
            fprintf(stderr, "HIP error: %s, in file: %s, line number: %d\n", hipGetErrorString(e_), \
                    __FILE__, __LINE__);                                                          \
            exit(1);                                                                              \
        }                                                                                         \
    } while (0)

static void die(const char *what) {
    OPENFISH_ERROR("%s", what);
    exit(EXIT_FAILURE);
}

static void launch_ok(int rc, const char *kernel) {
    if (rc == 0) return;
    if (rc == OFK_BAD_ARGS) fprintf(stderr, "openfish: %s: arguments do not fit the kernel (shape, alignment or state_len)\n", kernel);
    else fprintf(stderr, "HIP error: %s, launching %s\n", hipGetErrorString((hipError_t)rc), kernel);
    exit(1);
}

static void *host_alloc(size_t bytes) {
    void *p = malloc(bytes ? bytes : 1);
    if (!p) {
        fprintf(stderr, "openfish: out of host memory (%zu bytes)\n", bytes);
        exit(EXIT_FAILURE);
    }
    return p;
}

/* ---- table of log(1 + e^-gap) for the beam search's merges -------------------
 *
 * The CPU path folds two scores with log(1.0 + exp(-gap)) in double (reference
 * src/beam_search.c:43-47).  On the device that value is read off a piecewise
 * polynomial: per cell of width 1/4 the degree-8 interpolant through the Chebyshev
 * nodes, fitted here in long double.  The interpolation error is below 1e-15, far
 * under the 2^-46 at which a folded fp32 score could round differently.
 */

static void build_lse_table(double *tab) {
    const int n = OFK_LSE_COEFS; /* nodes = coefficients */
    const long double pi = 3.14159265358979323846264338327950288L;
    for (int cell = 0; cell < OFK_LSE_CELLS; ++cell) {
        const long double centre = 0.25L * cell + 0.125L;
        long double x[OFK_LSE_COEFS], dd[OFK_LSE_COEFS], mono[OFK_LSE_COEFS], basis[OFK_LSE_COEFS];
        for (int j = 0; j < n; ++j) {
            x[j] = cosl(pi * (2 * j + 1) / (2.0L * n)); /* s in [-1, 1], gap = centre + s / 8 */
            dd[j] = log1pl(expl(-(centre + x[j] / 8.0L)));
        }
        for (int k = 1; k < n; ++k) /* Newton divided differences */
            for (int j = n - 1; j >= k; --j) dd[j] = (dd[j] - dd[j - 1]) / (x[j] - x[j - k]);
        for (int j = 0; j < n; ++j) mono[j] = 0, basis[j] = 0;
        basis[0] = 1; /* basis = prod_{m<k} (s - x[m]) as monomials */
        for (int k = 0; k < n; ++k) {
            for (int j = 0; j < n; ++j) mono[j] += dd[k] * basis[j];
            for (int j = n - 1; j >= 1; --j) basis[j] = basis[j - 1] - x[k] * basis[j];
            basis[0] = -x[k] * basis[0];
        }
        for (int j = 0; j < n; ++j) tab[cell * n + j] = (double)mono[j];
    }
}

void openfish_amd_lse_table(double *out) { build_lse_table(out); }

/* ---- gpubuf ---------------------------------------------------------------- */

#define OFA_MAGIC 0x6f66616d64677075ull /* "ofamdgpu" */

enum { EV_JOIN, EV_START, EV_BWD_END, EV_BEAM_START, EV_BEAM_END, EV_FWD_END, EV_SEQ_START, EV_SEQ_END, EV_SUMS_START, EV_SUMS_END, EV_COUNT };
/* with both sweeps in one kernel EV_BWD_END marks its end and EV_FWD_END is not recorded */

typedef struct {
    openfish_gpubuf_t pub; /* first: the pointer handed to callers is this struct */
    unsigned long long magic;
    int T, N, state_len;
    void *slab;            /* one device allocation behind all pub fields */
    float *path_sums;      /* N x T x states: per state, the posteriors a block's quality is made of, summed */
    unsigned char *h_out;  /* pinned host memory for moves | sequence | qstring */
    unsigned char *d_out;  /* the same memory as the device addresses it */
    double *lse_table;     /* device copy of the log(1 + e^-gap) table */
    hipStream_t s_main, s_side;
    hipEvent_t ev[EV_COUNT];
    float ms[OPENFISH_AMD_STAGE_COUNT];
    int timed;
    int pending;           /* a decode has been enqueued and not yet waited for */
    int pend_T, pend_N, pend_sums;    /* its shape */
    int pend_split;        /* how its scans were queued (which events were recorded) */
    int scan_mode;         /* OFK_SCAN_*: arithmetic of the scans of this gpubuf's decodes */
    int scan_spl;          /* states per lane of the scans, 0 = chosen from the batch size */
    int debug_flags;       /* bit 0: serial replay of the beam search's merges; bit 1: colliding seed hashes */
    int split_scans;       /* 1: backward sweep, then forward sweep beside the beam search; 0: both sweeps in one
                            * kernel; -1 (default): chosen per call by split_by_default() */
    ofk_phred_table_t phred; /* thresholds for (phred_shift, phred_scale) */
    float phred_shift, phred_scale;
    int phred_valid;
} ofa_gpubuf_t;

static size_t round_up(size_t x) { return (x + 255) & ~(size_t)255; }

static int states_of(int state_len) { return 1 << (2 * state_len); }

static void check_state_len(int state_len) {
    if (state_len < 3 || state_len > 5) die("state_len must be 3, 4 or 5 (64, 256 or 1024 states)");
}

openfish_gpubuf_t *openfish_gpubuf_init(const int T, const int N, const int state_len) {
    check_state_len(state_len);
    if (T < 1 || N < 1) die("gpubuf: T and N must be positive");
    if (T > OFK_MAX_T) die("gpubuf: chunks longer than 8192 time steps are not supported");
    const size_t S = (size_t)states_of(state_len), nt = (size_t)N * (size_t)T;
    const size_t tens = sizeof(float) * (size_t)N * (size_t)(T + 1) * S;
    ofa_gpubuf_t *g = (ofa_gpubuf_t *)host_alloc(sizeof *g);
    memset(g, 0, sizeof *g);
    g->magic = OFA_MAGIC;
    g->T = T;
    g->N = N;
    g->state_len = state_len;
    g->split_scans = -1;

    /* field sizes as in the reference (src/decode_hip.hip:24-48) except beam_vector,
     * whose slots are 2 bytes here */
    const size_t sz[11] = {tens, tens, nt, nt, nt,
                           sizeof(ofk_beam_slot_t) * (size_t)N * OFK_BEAM_WIDTH * (size_t)(T + 1),
                           sizeof(int32_t) * nt, sizeof(float) * 4 * nt, sizeof(float) * nt, sizeof(float) * nt,
                           /* path_sums, not a field of the reference's struct; see enqueue_decode */
                           (state_len <= 4 ? sizeof(float) * S * (size_t)T * (size_t)(N < OFK_SPARSE_SEARCH_MAX_CHUNKS ? N : OFK_SPARSE_SEARCH_MAX_CHUNKS) : 0)};
    size_t total = 0;
    for (int i = 0; i < 11; ++i) total += round_up(sz[i]);
    HIP_OK(hipMalloc(&g->slab, total));
    unsigned char *p = (unsigned char *)g->slab;
    void **field[11] = {(void **)&g->pub.bwd_NTC, (void **)&g->pub.post_NTC, (void **)&g->pub.moves,
                        (void **)&g->pub.sequence, (void **)&g->pub.qstring, &g->pub.beam_vector,
                        &g->pub.states, (void **)&g->pub.qual_data, (void **)&g->pub.base_probs,
                        (void **)&g->pub.total_probs, (void **)&g->path_sums};
    for (int i = 0; i < 11; ++i) {
        *field[i] = sz[i] ? p : NULL;
        p += round_up(sz[i]);
    }
    HIP_OK(hipHostMalloc((void **)&g->h_out, 3 * nt, hipHostMallocDefault));
    HIP_OK(hipHostGetDevicePointer((void **)&g->d_out, g->h_out, 0));
    {
        double tab[OFK_LSE_DOUBLES];
        build_lse_table(tab);
        HIP_OK(hipMalloc((void **)&g->lse_table, sizeof tab));
        HIP_OK(hipMemcpy(g->lse_table, tab, sizeof tab, hipMemcpyHostToDevice));
    }
    HIP_OK(hipStreamCreateWithFlags(&g->s_main, hipStreamNonBlocking));
    HIP_OK(hipStreamCreateWithFlags(&g->s_side, hipStreamNonBlocking));
    for (int i = 0; i < EV_COUNT; ++i) HIP_OK(hipEventCreate(&g->ev[i]));
    return &g->pub;
}

void openfish_gpubuf_free(openfish_gpubuf_t *gpubuf) {
    ofa_gpubuf_t *g = (ofa_gpubuf_t *)gpubuf;
    if (!g) return;
    if (g->magic != OFA_MAGIC) die("gpubuf was not created by openfish_gpubuf_init");
    if (g->pending) { /* an enqueued decode still reads and writes these buffers */
        HIP_OK(hipStreamSynchronize(g->s_side));
        HIP_OK(hipStreamSynchronize(g->s_main));
    }
    for (int i = 0; i < EV_COUNT; ++i) HIP_OK(hipEventDestroy(g->ev[i]));
    HIP_OK(hipStreamDestroy(g->s_main));
    HIP_OK(hipStreamDestroy(g->s_side));
    HIP_OK(hipHostFree(g->h_out));
    HIP_OK(hipFree(g->lse_table));
    HIP_OK(hipFree(g->slab));
    g->magic = 0;
    free(g);
}

static ofa_gpubuf_t *checked(const openfish_gpubuf_t *gpubuf, int T, int N, int state_len) {
    ofa_gpubuf_t *g = (ofa_gpubuf_t *)gpubuf;
    if (!g || g->magic != OFA_MAGIC) die("gpubuf was not created by openfish_gpubuf_init");
    if (state_len != g->state_len || (size_t)N * (size_t)(T + 1) > (size_t)g->N * (size_t)(g->T + 1) ||
        (size_t)N * (size_t)T > (size_t)g->N * (size_t)g->T)
        die("batch shape exceeds the shape the gpubuf was created for");
    if (g->pending) die("this gpubuf holds an enqueued decode that has not been waited for");
    return g;
}

/* Scores carry, per state, the four step columns, or five with a blank/stay column first (as a
 * CRF head emits them before the blank is dropped).  The kernels read either layout where it
 * lies and never look at the blank column: the stay score is options->blank_score, as for any
 * other input (reference src/beam_search.c:213). */
static void check_scores(int T, int N, int C, const void *scores, int state_len, const openfish_opt_t *opt) {
    check_state_len(state_len);
    if (T < 1 || N < 1) die("T and N must be positive");
    if (T > OFK_MAX_T) die("chunks longer than 8192 time steps are not supported");
    if (C != 4 * states_of(state_len) && C != 5 * states_of(state_len))
        die("C must be 4 * 4^state_len (one score per state and dropped base) or 5 * 4^state_len (a blank "
            "column first)");
    if (!scores) die("scores_TNC is NULL");
    if (!opt) die("options is NULL");
}

static int columns_of(int C, int state_len) { return C / states_of(state_len); }

static float log_beam_cut(const openfish_opt_t *opt) {
    /* reference src/beam_search.c:135 */
    return opt->beam_cut > 0.0f ? logf(opt->beam_cut) : FLT_MAX;
}

/* ---- phred thresholds -------------------------------------------------------
 *
 * The quality character of a base is char(x) = (char)(33.5f + clamp(-10*log10f(x)*scale
 * + shift, 1, 50)) of its miss probability x = 1 - base_prob/total_prob (reference
 * src/beam_search.c:92-97).  log10f is a libm routine whose last bit a device routine
 * cannot be relied on to reproduce, but char(x) only steps 49 times over [0,1]: the
 * thresholds are located here by bisection over the float bit patterns with this
 * host's log10f, the neighbourhood of each is checked for monotonicity, and the
 * kernel compares x against them.
 */

static int phred_char(float x, float scale, float shift) {
    volatile float v = -10.0f * log10f(x);
    volatile float q = v * scale;
    q = q + shift;
    if (q > 50.0f) q = 50.0f;
    if (q < 1.0f) q = 1.0f;
    return (int)(char)(33.5f + q);
}

static float bits_float(uint32_t b) {
    float f;
    memcpy(&f, &b, sizeof f);
    return f;
}

static void build_phred_table(ofk_phred_table_t *tab, float scale, float shift) {
    const uint32_t one = 0x3f800000u; /* 1.0f; bit patterns of [0,1] are ordered like the values */
    for (int j = 0; j < OFK_PHRED_STEPS; ++j) {
        const int limit = 82 - j;
        if (phred_char(1.0f, scale, shift) > limit) {
            tab->thr[j] = 2.0f; /* never reached on [0,1] */
            continue;
        }
        uint32_t lo = 0, hi = one; /* char(lo) > limit >= char(hi) */
        if (phred_char(0.0f, scale, shift) <= limit) hi = 0;
        while (hi - lo > 1 && hi != 0) {
            const uint32_t mid = lo + (hi - lo) / 2;
            if (phred_char(bits_float(mid), scale, shift) <= limit) hi = mid;
            else lo = mid;
        }
        tab->thr[j] = bits_float(hi);
        for (uint32_t d = 1; d <= 64; ++d) {
            const int below = hi >= d ? phred_char(bits_float(hi - d), scale, shift) : 127;
            const int above = hi + d <= one ? phred_char(bits_float(hi + d), scale, shift) : 0;
            if (below <= limit || above > limit)
                die("phred character is not monotone in the miss probability near a threshold");
        }
    }
}

void openfish_amd_phred_table(float q_scale, float q_shift, float *thr49) {
    ofk_phred_table_t tab;
    build_phred_table(&tab, q_scale, q_shift);
    memcpy(thr49, tab.thr, sizeof tab.thr);
}

static const ofk_phred_table_t *phred_for(ofa_gpubuf_t *g, const openfish_opt_t *opt) {
    if (!g->phred_valid || g->phred_shift != opt->q_shift || g->phred_scale != opt->q_scale) {
        build_phred_table(&g->phred, opt->q_scale, opt->q_shift);
        g->phred_shift = opt->q_shift;
        g->phred_scale = opt->q_scale;
        g->phred_valid = 1;
    }
    return &g->phred;
}

/* ---- decode ---------------------------------------------------------------- */

/* The three result buffers are the caller's to free (the reference's contract), so they are fresh
 * allocations every call.  They are allocated and touched while the GPU works, which takes the page
 * faults off the path between the last kernel and the return. */
static void alloc_outputs(int T, int N, uint8_t **moves, char **sequence, char **qstring) {
    const size_t nt = (size_t)N * (size_t)T;
    *moves = (uint8_t *)host_alloc(nt);
    *sequence = (char *)host_alloc(nt);
    *qstring = (char *)host_alloc(nt);
    memset(*moves, 0, nt);
    memset(*sequence, 0, nt);
    memset(*qstring, 0, nt);
}

/* all three results over the main stream (the stage-level entry point) */
static void fetch_outputs(ofa_gpubuf_t *g, int T, int N, uint8_t **moves, char **sequence, char **qstring) {
    const size_t nt = (size_t)N * (size_t)T;
    HIP_OK(hipMemcpyAsync(g->h_out, g->pub.moves, nt, hipMemcpyDeviceToHost, g->s_main));
    HIP_OK(hipMemcpyAsync(g->h_out + nt, g->pub.sequence, nt, hipMemcpyDeviceToHost, g->s_main));
    HIP_OK(hipMemcpyAsync(g->h_out + 2 * nt, g->pub.qstring, nt, hipMemcpyDeviceToHost, g->s_main));
    alloc_outputs(T, N, moves, sequence, qstring);
    HIP_OK(hipStreamSynchronize(g->s_main));
    memcpy(*moves, g->h_out, nt);
    memcpy(*sequence, g->h_out + nt, nt);
    memcpy(*qstring, g->h_out + 2 * nt, nt);
}

/* order the library's streams after everything already queued on the null stream */
static void join_null_stream(ofa_gpubuf_t *g) {
    HIP_OK(hipEventRecord(g->ev[EV_JOIN], 0));
    HIP_OK(hipStreamWaitEvent(g->s_main, g->ev[EV_JOIN], 0));
}

/* Which arrangement of the scans a blocking decode finishes sooner with, as measured on whole
 * decodes (T = 1666; chunks/s with one kernel | split):
 *     64 states:  512 chunks 248k | 260k, 2048 chunks 418k | 485k
 *    256 states:  128 chunks  57k |  61k,  512 chunks 180k | 195k, 1024 chunks 215k | 206k, 2048 chunks 223k | 207k
 *   1024 states:   64 chunks 16.6k | 16.9k, 256 chunks 57.7k | 55.2k
 * Up to 512 chunks of 256 states (or as many states in all with 64 per chunk) the beam search, one
 * wave per chunk, is the longest stage and leaves most of the machine idle: the forward sweep and the
 * posterior fit beside it.  Beyond that the search fills the compute units itself and the one
 * kernel, which has the shorter scan stage at every size, wins. */
static int split_by_default(int N, int state_len) {
    return state_len <= 4 && (long)N * states_of(state_len) <= 512L * 256L;
}

/* Queue one decode on the gpubuf's streams, results into its pinned staging buffer; returns
 * without waiting for the GPU. */
static void enqueue_decode(ofa_gpubuf_t *g, const int T, const int N, const int C, const void *scores_TNC,
                           const int state_len, const openfish_opt_t *options) {
    const float stay = options->blank_score; /* as the reference GPU path, src/decode_hip.hip:120 */
    const size_t nt = (size_t)N * (size_t)T;

    join_null_stream(g);
    HIP_OK(hipEventRecord(g->ev[EV_START], g->s_main));
    const int cols = columns_of(C, state_len);
    g->pend_split = g->split_scans < 0 ? split_by_default(N, state_len) : g->split_scans;
    /* only where the search leaves the machine idle, and not with 1024 states, whose search waits for
     * memory and was measured to take half as long again beside the extra kernel */
    /* With split scans the posteriors are complete when the forward kernel ends.  With 64 states that is
     * well before the search does (0.83 against 1.13 ms at 512 chunks), and the sums (0.21 ms) fit in
     * between; with 256 states the two end together and the sequence stage gathers by itself. */
    const int sums_fit = g->path_sums != NULL && N <= OFK_SPARSE_SEARCH_MAX_CHUNKS;
    const int use_sums = sums_fit && (!g->pend_split || state_len == 3);
    g->pend_sums = use_sums;
    if (!g->pend_split) {
        /* both sweeps and the posterior in one kernel, then the beam search, all on one stream */
        launch_ok(ofk_scan_posterior(scores_TNC, g->pub.bwd_NTC, g->pub.post_NTC, T, N, state_len, cols, stay, g->scan_mode,
                                     g->scan_spl, g->s_main), "scan_posterior");
        HIP_OK(hipEventRecord(g->ev[EV_BWD_END], g->s_main));
        HIP_OK(hipEventRecord(g->ev[EV_BEAM_START], g->s_main));
        launch_ok(ofk_beam_search(scores_TNC, g->pub.bwd_NTC, (ofk_beam_slot_t *)g->pub.beam_vector,
                                  (int32_t *)g->pub.states, g->pub.moves, T, N, state_len, cols, log_beam_cut(options),
                                  stay, g->lse_table, g->debug_flags, g->s_main), "beam_search");
        HIP_OK(hipEventRecord(g->ev[EV_BEAM_END], g->s_main));
        /* The search keeps one wave per chunk busy and leaves the rest of the machine idle: beside
         * it, on the second stream, the posteriors that a block's quality is made of are summed for
         * every state, so that the sequence stage reads one value per time step instead of nine. */
        if (use_sums) {
            HIP_OK(hipStreamWaitEvent(g->s_side, g->ev[EV_BWD_END], 0));
            HIP_OK(hipEventRecord(g->ev[EV_SUMS_START], g->s_side));
            launch_ok(ofk_path_sums(g->pub.post_NTC, g->path_sums, T, N, state_len, g->s_side), "path_sums");
            HIP_OK(hipEventRecord(g->ev[EV_SUMS_END], g->s_side));
        }
        /* the moves are final once the beam search is: they travel while the sequence stage runs */
        HIP_OK(hipStreamWaitEvent(g->s_side, g->ev[EV_BEAM_END], 0));
        HIP_OK(hipMemcpyAsync(g->h_out, g->pub.moves, nt, hipMemcpyDeviceToHost, g->s_side));
        if (use_sums) HIP_OK(hipStreamWaitEvent(g->s_main, g->ev[EV_SUMS_END], 0));
    } else {
        launch_ok(ofk_bwd_scan(scores_TNC, g->pub.bwd_NTC, T, N, state_len, cols, stay, g->scan_mode, g->scan_spl, g->s_main),
                  "bwd_scan");
        HIP_OK(hipEventRecord(g->ev[EV_BWD_END], g->s_main));

        /* The beam search is the longer of the two stages that follow and wants its workgroups (large
         * LDS blocks) resident before the forward sweep fills the compute units: it stays on the stream
         * the backward sweep ran on and so starts first; the forward sweep follows through an event. */
        HIP_OK(hipEventRecord(g->ev[EV_BEAM_START], g->s_main));
        launch_ok(ofk_beam_search(scores_TNC, g->pub.bwd_NTC, (ofk_beam_slot_t *)g->pub.beam_vector,
                                  (int32_t *)g->pub.states, g->pub.moves, T, N, state_len, cols, log_beam_cut(options),
                                  stay, g->lse_table, g->debug_flags, g->s_main), "beam_search");
        HIP_OK(hipEventRecord(g->ev[EV_BEAM_END], g->s_main));

        HIP_OK(hipStreamWaitEvent(g->s_side, g->ev[EV_BWD_END], 0));
        launch_ok(ofk_fwd_post_scan(scores_TNC, g->pub.bwd_NTC, g->pub.post_NTC, T, N, state_len, cols, stay, g->scan_mode,
                                    g->scan_spl, g->s_side), "fwd_post_scan");
        HIP_OK(hipEventRecord(g->ev[EV_FWD_END], g->s_side));
        if (use_sums) {
            HIP_OK(hipEventRecord(g->ev[EV_SUMS_START], g->s_side));
            launch_ok(ofk_path_sums(g->pub.post_NTC, g->path_sums, T, N, state_len, g->s_side), "path_sums");
            HIP_OK(hipEventRecord(g->ev[EV_SUMS_END], g->s_side));
        }
        /* the moves are final once the beam search is: they travel while the sequence stage runs */
        HIP_OK(hipStreamWaitEvent(g->s_side, g->ev[EV_BEAM_END], 0));
        HIP_OK(hipMemcpyAsync(g->h_out, g->pub.moves, nt, hipMemcpyDeviceToHost, g->s_side));
        HIP_OK(hipStreamWaitEvent(g->s_main, g->ev[use_sums ? EV_SUMS_END : EV_FWD_END], 0));
    }

    HIP_OK(hipEventRecord(g->ev[EV_SEQ_START], g->s_main));
    /* The last kernel writes bases and qualities straight into the pinned host memory (N * T bytes
     * each, every byte once, 64 consecutive bytes per wave store): they are in host memory when the
     * kernel ends and no copy follows it, which measured 0.05 ms less per call at 512 x 1666 than two
     * copies after a kernel that is 0.03 ms shorter.  The gpubuf's own sequence and qstring arrays
     * are filled by the stage-level entry points only. */
    launch_ok(ofk_sequence(g->pub.post_NTC, (int32_t *)g->pub.states, g->pub.moves, g->pub.qual_data,
                           g->pub.base_probs, g->pub.total_probs, (char *)g->d_out + nt, (char *)g->d_out + 2 * nt, T, N,
                           state_len, phred_for(g, options), use_sums ? g->path_sums : NULL, g->s_main), "sequence");
    HIP_OK(hipEventRecord(g->ev[EV_SEQ_END], g->s_main));
    g->pending = 1;
    g->pend_T = T;
    g->pend_N = N;
}

void openfish_decode_gpu(const int T, const int N, const int C, void *scores_TNC, const int state_len,
                         const openfish_opt_t *options, const openfish_gpubuf_t *gpubuf, uint8_t **moves,
                         char **sequence, char **qstring) {
    check_scores(T, N, C, scores_TNC, state_len, options);
    if (!moves || !sequence || !qstring) die("decode: output pointer is NULL");
    ofa_gpubuf_t *g = checked(gpubuf, T, N, state_len);
    const size_t nt = (size_t)N * (size_t)T;
    OPENFISH_LOG_TRACE("scores tensor dim: %d, %d, %d", T, N, C);

    enqueue_decode(g, T, N, C, scores_TNC, state_len, options);
    alloc_outputs(T, N, moves, sequence, qstring);
    HIP_OK(hipStreamSynchronize(g->s_side));
    memcpy(*moves, g->h_out, nt);
    HIP_OK(hipStreamSynchronize(g->s_main));
    memcpy(*sequence, g->h_out + nt, nt);
    memcpy(*qstring, g->h_out + 2 * nt, nt);
    g->pending = 0;
    g->timed = 1;
}

void openfish_amd_decode_enqueue(int T, int N, int C, const void *scores_TNC, int state_len,
                                 const openfish_opt_t *options, const openfish_gpubuf_t *gpubuf) {
    check_scores(T, N, C, scores_TNC, state_len, options);
    ofa_gpubuf_t *g = checked(gpubuf, T, N, state_len);
    enqueue_decode(g, T, N, C, scores_TNC, state_len, options);
}

void openfish_amd_decode_wait(const openfish_gpubuf_t *gpubuf, const uint8_t **moves, const char **sequence,
                              const char **qstring) {
    ofa_gpubuf_t *g = (ofa_gpubuf_t *)gpubuf;
    if (!g || g->magic != OFA_MAGIC) die("gpubuf was not created by openfish_gpubuf_init");
    if (!g->pending) die("decode_wait: nothing was enqueued on this gpubuf");
    if (!moves || !sequence || !qstring) die("decode_wait: output pointer is NULL");
    const size_t nt = (size_t)g->pend_N * (size_t)g->pend_T;
    HIP_OK(hipStreamSynchronize(g->s_side));
    HIP_OK(hipStreamSynchronize(g->s_main));
    *moves = g->h_out;
    *sequence = (const char *)g->h_out + nt;
    *qstring = (const char *)g->h_out + 2 * nt;
    g->pending = 0;
    g->timed = 1;
}

int openfish_amd_last_timings(const openfish_gpubuf_t *gpubuf, float *ms, int n) {
    ofa_gpubuf_t *g = (ofa_gpubuf_t *)gpubuf;
    if (!g || g->magic != OFA_MAGIC) die("gpubuf was not created by openfish_gpubuf_init");
    if (!g->timed || !ms || n < 1) return 0;
    if (g->pend_split) {
        HIP_OK(hipEventElapsedTime(&g->ms[OPENFISH_AMD_STAGE_BWD], g->ev[EV_START], g->ev[EV_BWD_END]));
        HIP_OK(hipEventElapsedTime(&g->ms[OPENFISH_AMD_STAGE_FWD], g->ev[EV_BWD_END], g->ev[EV_FWD_END]));
        g->ms[OPENFISH_AMD_STAGE_SCAN] = 0.0f;
    } else {
        g->ms[OPENFISH_AMD_STAGE_BWD] = g->ms[OPENFISH_AMD_STAGE_FWD] = 0.0f;
        HIP_OK(hipEventElapsedTime(&g->ms[OPENFISH_AMD_STAGE_SCAN], g->ev[EV_START], g->ev[EV_BWD_END]));
    }
    HIP_OK(hipEventElapsedTime(&g->ms[OPENFISH_AMD_STAGE_BEAM], g->ev[EV_BEAM_START], g->ev[EV_BEAM_END]));
    HIP_OK(hipEventElapsedTime(&g->ms[OPENFISH_AMD_STAGE_SEQ], g->ev[EV_SEQ_START], g->ev[EV_SEQ_END]));
    HIP_OK(hipEventElapsedTime(&g->ms[OPENFISH_AMD_STAGE_TOTAL], g->ev[EV_START], g->ev[EV_SEQ_END]));
    g->ms[OPENFISH_AMD_STAGE_SUMS] = 0.0f;
    if (g->pend_sums) HIP_OK(hipEventElapsedTime(&g->ms[OPENFISH_AMD_STAGE_SUMS], g->ev[EV_SUMS_START], g->ev[EV_SUMS_END]));
    if (n > OPENFISH_AMD_STAGE_COUNT) n = OPENFISH_AMD_STAGE_COUNT;
    memcpy(ms, g->ms, sizeof(float) * (size_t)n);
    return n;
}

/* ---- stages ---------------------------------------------------------------- */

static void check_scan_mode(int scan_mode) {
    if (scan_mode != OFK_SCAN_TWO_TIER && scan_mode != OFK_SCAN_PRECISE && scan_mode != OFK_SCAN_FAST)
        die("scan mode must be OPENFISH_AMD_SCAN_TWO_TIER, _PRECISE or _FAST");
}

void openfish_amd_bwd_scan(int T, int N, int C, const void *scores, int state_len, float stay_score, int scan_mode,
                           float *bwd) {
    openfish_opt_t o = DECODER_INIT;
    check_scores(T, N, C, scores, state_len, &o);
    check_scan_mode(scan_mode);
    launch_ok(ofk_bwd_scan(scores, bwd, T, N, state_len, columns_of(C, state_len), stay_score, scan_mode, 0, NULL), "bwd_scan");
    HIP_OK(hipStreamSynchronize(0));
}

void openfish_amd_fwd_post_scan(int T, int N, int C, const void *scores, int state_len, float stay_score,
                                int scan_mode, const float *bwd, float *post) {
    openfish_opt_t o = DECODER_INIT;
    check_scores(T, N, C, scores, state_len, &o);
    check_scan_mode(scan_mode);
    launch_ok(ofk_fwd_post_scan(scores, bwd, post, T, N, state_len, columns_of(C, state_len), stay_score, scan_mode, 0, NULL), "fwd_post_scan");
    HIP_OK(hipStreamSynchronize(0));
}

void openfish_amd_scan_posterior(int T, int N, int C, const void *scores, int state_len, float stay_score,
                                 int scan_mode, float *bwd, float *post) {
    openfish_opt_t o = DECODER_INIT;
    check_scores(T, N, C, scores, state_len, &o);
    check_scan_mode(scan_mode);
    launch_ok(ofk_scan_posterior(scores, bwd, post, T, N, state_len, columns_of(C, state_len), stay_score, scan_mode, 0, NULL), "scan_posterior");
    HIP_OK(hipStreamSynchronize(0));
}

void openfish_amd_beam_search(int T, int N, int C, const void *scores, int state_len,
                              const openfish_opt_t *options, const float *bwd, const openfish_gpubuf_t *gpubuf) {
    check_scores(T, N, C, scores, state_len, options);
    ofa_gpubuf_t *g = checked(gpubuf, T, N, state_len);
    launch_ok(ofk_beam_search(scores, bwd, (ofk_beam_slot_t *)g->pub.beam_vector, (int32_t *)g->pub.states,
                              g->pub.moves, T, N, state_len, columns_of(C, state_len), log_beam_cut(options),
                              options->blank_score,
                              g->lse_table, g->debug_flags, NULL),
              "beam_search");
    HIP_OK(hipStreamSynchronize(0));
}

void openfish_amd_beam_search_static_prepare(void) {
    if (ofk_beam_search_static_ready()) return;
    double tab[OFK_LSE_DOUBLES];
    build_lse_table(tab);
    launch_ok(ofk_beam_search_static_prepare(tab), "beam_search_static_prepare");
}

void openfish_amd_beam_search_static(int T, int N, int C, const void *scores, int state_len,
                                     const openfish_opt_t *options, const float *bwd, int32_t *states,
                                     uint8_t *moves, void *stream) {
    check_scores(T, N, C, scores, state_len, options);
    if (!bwd || !states || !moves) die("beam_search_static: bwd, states and moves must be device pointers");
    const int rc = ofk_beam_search_static(scores, bwd, states, moves, T, N, state_len, columns_of(C, state_len),
                                          log_beam_cut(options), options->blank_score, 0, stream);
    if (rc == OFK_NOT_PREPARED)
        die("beam_search_static: call openfish_amd_beam_search_static_prepare() on this device first");
    if (rc == OFK_TOO_LARGE) {
        fprintf(stderr, "openfish: beam_search_static: N * (T + 1) * 64 = %zu bytes of beam slots exceed the static "
                        "scratch array of %u bytes; use openfish_amd_beam_search with a gpubuf\n",
                (size_t)N * (size_t)(T + 1) * 64, (unsigned)OFK_STATIC_SLOT_BYTES);
        exit(EXIT_FAILURE);
    }
    launch_ok(rc, "beam_search_static");
}

size_t openfish_amd_device_free_bytes(void) {
    size_t free_b = 0, total_b = 0;
    HIP_OK(hipMemGetInfo(&free_b, &total_b));
    return free_b;
}

void openfish_amd_sequence(int T, int N, int state_len, const openfish_opt_t *options, const float *post,
                           const openfish_gpubuf_t *gpubuf) {
    if (!options) die("options is NULL");
    ofa_gpubuf_t *g = checked(gpubuf, T, N, state_len);
    launch_ok(ofk_sequence(post, (int32_t *)g->pub.states, g->pub.moves, g->pub.qual_data, g->pub.base_probs,
                           g->pub.total_probs, g->pub.sequence, g->pub.qstring, T, N, state_len,
                           phred_for(g, options), NULL, NULL), "sequence");
    HIP_OK(hipStreamSynchronize(0));
}

void openfish_amd_decode_from_tensors(int T, int N, int C, const void *scores, int state_len,
                                      const openfish_opt_t *options, const float *bwd, const float *post,
                                      const openfish_gpubuf_t *gpubuf, uint8_t **moves, char **sequence,
                                      char **qstring) {
    check_scores(T, N, C, scores, state_len, options);
    if (!moves || !sequence || !qstring) die("decode: output pointer is NULL");
    ofa_gpubuf_t *g = checked(gpubuf, T, N, state_len);
    join_null_stream(g);
    launch_ok(ofk_beam_search(scores, bwd, (ofk_beam_slot_t *)g->pub.beam_vector, (int32_t *)g->pub.states,
                              g->pub.moves, T, N, state_len, columns_of(C, state_len), log_beam_cut(options),
                              options->blank_score,
                              g->lse_table, g->debug_flags, g->s_main), "beam_search");
    /* the quality stage as a whole decode runs it: from per-state sums where the gpubuf holds room for them */
    const float *sums = NULL;
    if (g->path_sums != NULL && N <= OFK_SPARSE_SEARCH_MAX_CHUNKS) {
        launch_ok(ofk_path_sums(post, g->path_sums, T, N, state_len, g->s_main), "path_sums");
        sums = g->path_sums;
    }
    launch_ok(ofk_sequence(post, (int32_t *)g->pub.states, g->pub.moves, g->pub.qual_data, g->pub.base_probs,
                           g->pub.total_probs, g->pub.sequence, g->pub.qstring, T, N, state_len,
                           phred_for(g, options), sums, g->s_main), "sequence");
    fetch_outputs(g, T, N, moves, sequence, qstring);
}

/* ---- rotary embedding ------------------------------------------------------ */

void openfish_rotary_emb_gpu(void *x_gpu, void *sin_gpu, void *cos_gpu, int batch_size, int seqlen, int nheads,
                             int head_dim, int rotary_half, int stride_batch, int stride_seq, int stride_head) {
    (void)head_dim; /* unused by the reference as well (src/rotary_emb_hip.h:36-45) */
    launch_ok(ofk_rotary_emb(x_gpu, (const float *)sin_gpu, (const float *)cos_gpu, batch_size, seqlen, nheads,
                             rotary_half, stride_batch, stride_seq, stride_head, NULL), "rotary_emb");
    HIP_OK(hipStreamSynchronize(0));
}

/* ---- CPU entry points of the reference API: not carried by this library ---- */

void openfish_decode_cpu(const int T, const int N, const int C, int nthreads, void *scores_TNC,
                         const int state_len, const openfish_opt_t *options, uint8_t **moves, char **sequence,
                         char **qstring) {
    (void)T; (void)N; (void)C; (void)nthreads; (void)scores_TNC; (void)state_len; (void)options;
    (void)moves; (void)sequence; (void)qstring;
    die("openfish_decode_cpu: this library carries the GPU path only");
}

void openfish_rotary_emb_cpu(void *x, void *sin_buf, void *cos_buf, int batch_size, int seqlen, int nheads,
                             int head_dim, int rotary_half, int stride_batch, int stride_seq, int stride_head,
                             int nthreads) {
    (void)x; (void)sin_buf; (void)cos_buf; (void)batch_size; (void)seqlen; (void)nheads; (void)head_dim;
    (void)rotary_half; (void)stride_batch; (void)stride_seq; (void)stride_head; (void)nthreads;
    die("openfish_rotary_emb_cpu: this library carries the GPU path only");
}

/* ---- device helpers -------------------------------------------------------- */

void set_device_hip(int device) { HIP_OK(hipSetDevice(device)); }

void *upload_scores_to_hip(const int T, const int N, const int C, const void *scores_TNC) {
    void *dev = NULL;
    const size_t bytes = 2 * (size_t)T * (size_t)N * (size_t)C;
    HIP_OK(hipMalloc(&dev, bytes));
    HIP_OK(hipMemcpy(dev, scores_TNC, bytes, hipMemcpyHostToDevice));
    return dev;
}

void free_scores_hip(void *scores_TNC_gpu) { HIP_OK(hipFree(scores_TNC_gpu)); }

static void dump_blob(const char *name, const void *dev, size_t bytes) {
    void *host = host_alloc(bytes);
    HIP_OK(hipMemcpy(host, dev, bytes, hipMemcpyDeviceToHost));
    FILE *fp = fopen(name, "w");
    if (!fp || fwrite(host, 1, bytes, fp) != bytes) {
        fprintf(stderr, "openfish: error writing %s: %s\n", name, strerror(errno));
        exit(EXIT_FAILURE);
    }
    fclose(fp);
    free(host);
}

void write_gpubuf_hip(const uint64_t T, const uint64_t N, const int state_len, const openfish_gpubuf_t *gpubuf) {
    check_state_len(state_len);
    const size_t S = (size_t)states_of(state_len), tens = sizeof(float) * N * (T + 1) * S, nt = N * T;
    dump_blob("bwd_NTC.blob", gpubuf->bwd_NTC, tens);
    dump_blob("post_NTC.blob", gpubuf->post_NTC, tens);
    dump_blob("qual_data.blob", gpubuf->qual_data, sizeof(float) * 4 * nt);
    dump_blob("base_probs.blob", gpubuf->base_probs, sizeof(float) * nt);
    dump_blob("total_probs.blob", gpubuf->total_probs, sizeof(float) * nt);
}

void *openfish_amd_malloc(size_t bytes) {
    void *dev = NULL;
    HIP_OK(hipMalloc(&dev, bytes ? bytes : 1));
    return dev;
}
void openfish_amd_free(void *dev) { HIP_OK(hipFree(dev)); }
void openfish_amd_memcpy_h2d(void *dev, const void *host, size_t bytes) { HIP_OK(hipMemcpy(dev, host, bytes, hipMemcpyHostToDevice)); }
void openfish_amd_memcpy_d2h(void *host, const void *dev, size_t bytes) { HIP_OK(hipMemcpy(host, dev, bytes, hipMemcpyDeviceToHost)); }
void openfish_amd_memset(void *dev, int value, size_t bytes) { HIP_OK(hipMemset(dev, value, bytes)); }
void openfish_amd_sync(void) { HIP_OK(hipDeviceSynchronize()); }
void openfish_amd_copy(void *dst, const void *src, size_t bytes) {
    launch_ok(ofk_copy(dst, src, bytes, NULL), "copy");
    HIP_OK(hipStreamSynchronize(0));
}

void openfish_amd_probe_hw_math(double *errors4, unsigned int *identities) {
    if (!errors4 || !identities) die("probe_hw_math: output pointer is NULL");
    void *dev = NULL;
    unsigned char host[40];
    HIP_OK(hipMalloc(&dev, sizeof host));
    launch_ok(ofk_probe_hw_math(dev, NULL), "probe_hw_math");
    HIP_OK(hipStreamSynchronize(0));
    HIP_OK(hipMemcpy(host, dev, sizeof host, hipMemcpyDeviceToHost));
    HIP_OK(hipFree(dev));
    memcpy(errors4, host, 4 * sizeof(double));
    memcpy(identities, host + 32, sizeof *identities);
    for (int k = 0; k < 4; ++k) errors4[k] *= 16777216.0; /* in units of 2^-24 */
}

int openfish_amd_device_count(void) {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) {
        (void)hipGetLastError();
        return 0;
    }
    return n;
}

/* Settings live in the gpubuf and are read when a decode is enqueued on it, so callers with one
 * gpubuf each (one per host thread) do not see each other's settings. */
static ofa_gpubuf_t *owned(const openfish_gpubuf_t *gpubuf) {
    ofa_gpubuf_t *g = (ofa_gpubuf_t *)gpubuf;
    if (!g || g->magic != OFA_MAGIC) die("gpubuf was not created by openfish_gpubuf_init");
    return g;
}

void openfish_amd_gpubuf_set_debug_flags(const openfish_gpubuf_t *gpubuf, int flags) {
    owned(gpubuf)->debug_flags = flags & 3;
}

void openfish_amd_gpubuf_set_scan_mode(const openfish_gpubuf_t *gpubuf, int scan_mode) {
    check_scan_mode(scan_mode);
    owned(gpubuf)->scan_mode = scan_mode;
}

void openfish_amd_gpubuf_set_split_scans(const openfish_gpubuf_t *gpubuf, int split) {
    owned(gpubuf)->split_scans = split < 0 ? -1 : (split ? 1 : 0);
}

void openfish_amd_gpubuf_set_scan_states_per_lane(const openfish_gpubuf_t *gpubuf, int spl) {
    if (spl != 0 && spl != 1 && spl != 2 && spl != 4) die("states per lane must be 0 (automatic), 1, 2 or 4");
    owned(gpubuf)->scan_spl = spl;
}

const char *openfish_amd_version(void) { return "openfish-amd gfx950"; }
