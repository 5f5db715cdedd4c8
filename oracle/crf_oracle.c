/*
 * CPU oracle: plain-C restatement of the reference CRF-CTC decode path.
 * TEST INFRASTRUCTURE ONLY (see crf_oracle.h for what pins each function).
 *
 * Build without FMA contraction and without -march flags so that every fp32
 * operation rounds exactly as in the reference's `gcc -O2` x86-64 build.
 */
#include "crf_oracle.h"

#include <float.h>
#include <math.h>
#include <pthread.h>
#include <stdlib.h>
#include <string.h>

/* The CPU scans ignore opt->blank_score and add the literal 2.0f for a stay (src/decode_cpu.c:14,56);
 * the reference's GPU scans add opt->blank_score (src/decode_hip.hip:120).  The default below is the
 * CPU path's; ofo_set_scan_stay is a test knob that puts another value in its place, so that the
 * GPU scans can be compared at other blank scores. */
static float g_scan_stay = 2.0f;
#define STAY_SCORE_SCAN g_scan_stay
void ofo_set_scan_stay(float stay) { g_scan_stay = stay; }
#define CRC_POLY 0x82f63b78u /* reflected Castagnoli polynomial */
#define CRC_SEED 0x12345678u /* src/decode.h:54 */

/* ---- small helpers ------------------------------------------------------ */

/* bitwise CRC-32C update, LSB first, no pre/post inversion (src/beam_search.c:103-115) */
uint32_t ofo_crc32c(uint32_t crc, uint32_t bits, int nbits) {
    while (nbits-- > 0) {
        uint32_t feed = (bits ^ crc) & 1u;
        crc >>= 1;
        if (feed) crc ^= CRC_POLY;
        bits >>= 1;
    }
    return crc;
}

/* one descending partition pass around v[lo]; returns the pivot's final slot
 * (src/beam_search.c:13-28) */
static int split_desc(float *v, int lo, int hi) {
    const float pivot = v[lo];
    int a = lo + 1, b = hi;
    while (a <= b) {
        if (v[a] < pivot && v[b] > pivot) {
            float t = v[a]; v[a] = v[b]; v[b] = t;
            ++a; --b;
        }
        if (v[a] >= pivot) ++a;
        if (v[b] <= pivot) --b;
    }
    { float t = v[lo]; v[lo] = v[b]; v[b] = t; }
    return b;
}

/* value of rank k (0 = largest) by quick-select; reorders v (src/beam_search.c:30-41) */
float ofo_kth_largest(float *v, int k, int n) {
    int lo = 0, hi = n - 1;
    for (;;) {
        int p = split_desc(v, lo, hi);
        if (p == k) return v[p];
        if (p < k) lo = p + 1; else hi = p - 1;
    }
}

/* log(e^x + e^y); the correction is evaluated in double and dropped once the
 * gap reaches 17 (src/beam_search.c:43-47) */
float ofo_log_sum_exp(float x, float y) {
    float gap = fabsf(x - y);
    float top = x > y ? x : y;
    if (gap < 17.0f) return (float)((double)top + log(1.0 + exp(-(double)gap)));
    return (float)((double)top + (double)0.0f);
}

/* max + log(sum exp(v - max)) over five fp32 values: fp32 differences, double
 * exp, fp32 running sum, double log, one rounding at the end
 * (src/decode_cpu.c:45-49 and :104-108) */
static inline float lse5(const float v[5], float vmax) {
    float acc = 0.0f;
    for (int i = 0; i < 5; ++i) acc = (float)((double)acc + exp((double)(v[i] - vmax)));
    return (float)((double)vmax + log((double)acc));
}

/* ---- scans -------------------------------------------------------------- */

/* bwd[t][s] for t = T..0 of one chunk (src/decode_cpu.c:13-52).
 * From state s the four successors are (4s mod S)+b; the transition score sits
 * at index succ*4 + (4s div S) of the time step's row. */
void ofo_backward_scan(const float *scores, float *bwd, size_t chunk, size_t T, size_t N, size_t S) {
    const size_t row = 4 * S;
    const float *in = scores + chunk * row;
    float *out = bwd + chunk * (T + 1) * S;

    for (size_t s = 0; s < S; ++s) out[T * S + s] = 0.0f;

    for (size_t t = T; t-- > 0;) {
        const float *sc = in + t * N * row;
        const float *nxt = out + (t + 1) * S;
        float *cur = out + t * S;
        for (size_t s = 0; s < S; ++s) {
            const size_t succ0 = (4 * s) % S;
            const size_t lead = (4 * s) / S;
            float v[5];
            v[0] = nxt[s] + STAY_SCORE_SCAN;
            float vmax = v[0];
            for (size_t b = 0; b < 4; ++b) {
                v[b + 1] = nxt[succ0 + b] + sc[(succ0 + b) * 4 + lead];
                if (!(vmax > v[b + 1])) vmax = v[b + 1];
            }
            cur[s] = lse5(v, vmax);
        }
    }
}

/* forward recursion; what is stored is fwd[t][s] + bwd[t][s] for t = 0..T
 * (src/decode_cpu.c:54-119).  Into state s the four predecessors are
 * s/4 + b*S/4 with score index 4s+b. */
void ofo_forward_scan(const float *scores, const float *bwd, float *fwd, size_t chunk, size_t T, size_t N, size_t S) {
    const size_t row = 4 * S;
    const size_t quarter = S / 4;
    const float *in = scores + chunk * row;
    float ping[2][OFO_MAX_STATES];

    for (size_t s = 0; s < S; ++s) ping[0][s] = 0.0f;

    for (size_t t = 0; t <= T; ++t) {
        const float *sc = in + t * N * row; /* not dereferenced at t == T */
        const float *cur = ping[t & 1];
        float *nxt = ping[(t & 1) ^ 1];
        const size_t base = (chunk * (T + 1) + t) * S;
        for (size_t s = 0; s < S; ++s) {
            float v[5];
            v[0] = cur[s] + STAY_SCORE_SCAN;
            float vmax = v[0];
            for (size_t b = 0; b < 4; ++b) {
                float step = t < T ? sc[4 * s + b] : 0.0f;
                v[b + 1] = cur[s / 4 + b * quarter] + step;
                if (!(vmax > v[b + 1])) vmax = v[b + 1];
            }
            nxt[s] = lse5(v, vmax);
            fwd[base + s] = cur[s] + bwd[base + s];
        }
    }
}

/* per time step softmax over states: double exp rounded to fp32, fp32 running
 * sum in state order, fp32 division (src/decode_cpu.c:121-147) */
void ofo_softmax(const float *fwd, float *post, size_t chunk, size_t T, size_t S) {
    float e[OFO_MAX_STATES];
    for (size_t t = 0; t <= T; ++t) {
        const float *in = fwd + (chunk * (T + 1) + t) * S;
        float *out = post + (chunk * (T + 1) + t) * S;
        float vmax = in[0];
        for (size_t s = 0; s < S; ++s) if (!(vmax > in[s])) vmax = in[s];
        float total = 0.0f;
        for (size_t s = 0; s < S; ++s) {
            e[s] = (float)exp((double)(in[s] - vmax));
            total += e[s];
        }
        for (size_t s = 0; s < S; ++s) out[s] = e[s] / total;
    }
}

/* ---- beam search -------------------------------------------------------- */

typedef struct {
    uint32_t hash;
    int32_t state;
    uint8_t prev;
    uint8_t stay;
} front_t;

static size_t count_at_least(const float *v, size_t n, float thr) {
    size_t c = 0;
    for (size_t i = 0; i < n; ++i) if (v[i] >= thr) ++c;
    return c;
}

/* Test knob, not part of the algorithm: seed hashes are taken from (state & mask), so that with a
 * narrow mask different sequences share hashes from the first block on and the duplicate-hash
 * branches of the merge loop (several equal hashes, a step matched by two stays) are exercised.
 * The default mask keeps every bit, which is the reference's seeding (src/beam_search.c:151-175). */
static uint32_t g_seed_state_mask = 0xFFFFFFFFu;
void ofo_set_seed_state_mask(uint32_t mask) { g_seed_state_mask = mask; }

void ofo_beam_search(const float *scores, size_t row_stride, const float *bwd, const float *post,
                     int state_bits, size_t T, float beam_cut, float stay_score,
                     int32_t *states, uint8_t *moves, float *qual_data,
                     ofo_beam_slot_t *beam, int32_t *path_states) {
    const size_t S = (size_t)1 << state_bits;
    const int32_t mask = (int32_t)(S - 1);
    const float log_cut = beam_cut > 0.0f ? logf(beam_cut) : FLT_MAX; /* src/beam_search.c:135 */
    const size_t W = OFO_BEAM_WIDTH;

    front_t cand[OFO_MAX_CANDIDATES], front[OFO_MAX_CANDIDATES];
    float cand_score[OFO_MAX_CANDIDATES], front_score[OFO_MAX_CANDIDATES];
    memset(front, 0, sizeof front);
    memset(front_score, 0, sizeof front_score);

    /* seeding: the W best states of bwd[0], taken in ascending state order (:151-175) */
    float seed_thr = -FLT_MAX;
    if (W < S) {
        float tmp[OFO_MAX_STATES];
        memcpy(tmp, bwd, S * sizeof(float));
        seed_thr = ofo_kth_largest(tmp, (int)W - 1, (int)S);
    }
    {
        size_t slot = 0;
        for (size_t s = 0; s < S && slot < W; ++s) {
            if (bwd[s] >= seed_thr) {
                front[slot].hash = ofo_crc32c(CRC_SEED, (uint32_t)s & g_seed_state_mask, 32);
                front[slot].state = (int32_t)s;
                front[slot].prev = 0;
                front[slot].stay = 0;
                front_score[slot] = 0.0f;
                ++slot;
            }
        }
    }
    size_t width = W < S ? W : S;
    for (size_t i = 0; i < width; ++i) {
        beam[i].state = front[i].state;
        beam[i].prev = front[i].prev;
        beam[i].stay = front[i].stay;
    }

    for (size_t t = 0; t < T; ++t) {
        const float *row = scores + t * row_stride;
        const float *guide = bwd + (t + 1) * S;
        float best = -FLT_MAX;
        size_t n = 0;

        /* step candidates, index 4*i+b (:205-256) */
        for (size_t i = 0; i < width; ++i) {
            const int32_t shifted = front[i].state << 2;
            for (int b = 0; b < 4; ++b) {
                const int32_t ns = (shifted & mask) | b;
                const int32_t idx = (ns << 2) + (shifted >> state_bits);
                const float trans = row[idx] * 1.0f;
                const float sc = front_score[i] + trans + guide[ns];
                cand[n].hash = ofo_crc32c(front[i].hash, (uint32_t)b, 2);
                cand[n].state = ns;
                cand[n].prev = (uint8_t)i;
                cand[n].stay = 0;
                cand_score[n] = sc;
                if (!(best > sc)) best = sc;
                ++n;
            }
        }

        /* stay candidates, index 4*width+i, merged with the step that spells the
         * same sequence (equal hash) (:258-318).  The reference guards the inner
         * loop with a one-probe presence filter over the step hashes; an equal
         * hash always passes that filter, so it is not restated here. */
        for (size_t i = 0; i < width; ++i) {
            const float sc = front_score[i] + stay_score + guide[front[i].state];
            const size_t me = n;
            cand[me].hash = front[i].hash;
            cand[me].state = front[i].state;
            cand[me].prev = (uint8_t)i;
            cand[me].stay = 1;
            cand_score[me] = sc;
            if (!(best > sc)) best = sc;

            const int last_base = front[i].state & 3;
            for (size_t j = 0; j < width; ++j) {
                const size_t st = (j << 2) | (size_t)last_base;
                if (cand[me].hash == cand[st].hash) {
                    const float folded = ofo_log_sum_exp(cand_score[me], cand_score[st]);
                    if (cand_score[me] > cand_score[st]) {
                        cand_score[me] = folded;
                        cand_score[st] = -FLT_MAX;
                    } else {
                        cand_score[st] = folded;
                        cand_score[me] = -FLT_MAX;
                    }
                    if (folded > best) best = folded;
                }
            }
            ++n;
        }

        /* cut-off: beam_cut below the best score, then bisect until 25..32
         * survive, at most 9 refinements (:320-381) */
        float cut = best - log_cut;
        size_t kept = count_at_least(cand_score, n, cut);
        if (kept > W) {
            const size_t min_keep = (W * 8) / 10;
            float lo = cut, hi = best;
            int guesses = 1;
            while ((kept > W || kept < min_keep) && guesses < 10) {
                if (kept > W) { lo = cut; cut = (cut + hi) / 2.0f; }
                else          { hi = cut; cut = (cut + lo) / 2.0f; }
                kept = count_at_least(cand_score, n, cut);
                ++guesses;
            }
            if (guesses == 10) {
                cut = hi;
                kept = count_at_least(cand_score, n, cut);
            }
            if (kept > W) kept = W;
        }

        /* survivors in candidate order, first W of them (:383-394) */
        {
            size_t w = 0;
            for (size_t r = 0; r < n && w < W; ++r) {
                if (cand_score[r] >= cut) {
                    front[w] = cand[r];
                    front_score[w] = cand_score[r];
                    ++w;
                }
            }
        }

        /* final block: best survivor into slot 0 (:398-414) */
        if (t == T - 1) {
            float top = -FLT_MAX;
            size_t arg = 0;
            for (size_t i = 0; i < kept; ++i) if (front_score[i] > top) { top = front_score[i]; arg = i; }
            front_t tf = front[0]; front[0] = front[arg]; front[arg] = tf;
            float ts = front_score[0]; front_score[0] = front_score[arg]; front_score[arg] = ts;
        }

        /* drop the guide term again and persist (:417-427) */
        for (size_t i = 0; i < kept; ++i) {
            front_score[i] -= guide[front[i].state];
            ofo_beam_slot_t *slot = &beam[(t + 1) * W + i];
            slot->state = front[i].state;
            slot->prev = front[i].prev;
            slot->stay = front[i].stay;
        }
        width = kept;
    }

    /* traceback from slot 0 of the last block (:432-439) */
    {
        uint8_t slot = 0;
        for (size_t t = T; t != 0; --t) {
            const ofo_beam_slot_t *e = &beam[t * W + slot];
            states[t - 1] = e->state;
            moves[t - 1] = e->stay ? 0 : 1;
            slot = e->prev;
        }
        moves[0] = 1;
    }

    /* per-block quality: posterior of the path k-mer plus its distinct one-base
     * shifts, to the power 0.4 (:441-496) */
    const int quarter = (int)S >> 2;
    for (size_t t = 0; t < T; ++t) {
        const int st = states[t];
        if (path_states) path_states[t] = st;
        const int base = st % 4;
        states[t] = base;
        const float *p = post + (t + 1) * S;
        float prob = p[st] * 1.0f;
        int nb[8];
        for (int b = 0; b < 4; ++b) {
            nb[2 * b] = (st >> 2) + quarter * b;
            nb[2 * b + 1] = (int)((size_t)(st << 2) % S) + b;
        }
        for (int k = 0; k < 8; ++k) {
            int fresh = nb[k] != st;
            for (int m = 0; fresh && m < k; ++m) if (nb[m] == nb[k]) fresh = 0;
            if (fresh) prob += p[nb[k]] * 1.0f;
        }
        if (prob > 1.0f) prob = 1.0f;
        else if (prob < 0.0f) prob = 0.0f;
        prob = powf(prob, 0.4f);
        const float other = (1.0f - prob) / 3.0f;
        for (int b = 0; b < 4; ++b) qual_data[t * 4 + b] = (b == base) ? prob : other;
    }
}

/* moves + per-block quality -> bases and phred characters (src/beam_search.c:49-99) */
void ofo_generate_sequence(const uint8_t *moves, const int32_t *states, const float *qual_data,
                           float shift, float scale, size_t T, size_t seq_len,
                           float *base_probs, float *total_probs, char *sequence, char *qstring) {
    static const char letters[4] = {'A', 'C', 'G', 'T'};
    size_t pos = 0;
    for (size_t t = 0; t < T; ++t) {
        const int base = states[t] & 3;
        const int mv = moves[t];
        const int at = (int)pos + (t == 0 ? 0 : mv - 1);
        base_probs[at] += qual_data[t * 4 + base];
        for (int k = 0; k < 4; ++k) total_probs[at] += qual_data[t * 4 + k];
        const int emit = (t == 0) ? 1 : mv;
        for (int j = 0; j < emit; ++j) sequence[pos++] = (char)base;
    }
    for (size_t i = 0; i < seq_len; ++i) {
        sequence[i] = letters[(int)sequence[i]];
        base_probs[i] = 1.0f - (base_probs[i] / total_probs[i]);
        base_probs[i] = -10.0f * log10f(base_probs[i]);
        float q = base_probs[i] * scale + shift;
        if (q > 50.0f) q = 50.0f;
        if (q < 1.0f) q = 1.0f;
        qstring[i] = (char)(33.5f + q);
    }
}

/* ---- threaded driver (src/decode_cpu.c:149-332) -------------------------- */

typedef struct {
    int T, N, C, state_len, first, last;
    const float *scores;
    const ofo_opt_t *opt;
    float *bwd, *fwd, *post;
    const float *bwd_in, *post_in;
    int32_t *states, *path_states;
    uint8_t *moves;
    float *qual, *base_probs, *total_probs;
    char *sequence, *qstring;
    ofo_beam_slot_t *beam;
} job_t;

static void *scan_worker(void *p) {
    job_t *j = (job_t *)p;
    const size_t S = (size_t)1 << (2 * j->state_len);
    for (int c = j->first; c < j->last; ++c) {
        ofo_backward_scan(j->scores, j->bwd, (size_t)c, (size_t)j->T, (size_t)j->N, S);
        ofo_forward_scan(j->scores, j->bwd, j->fwd, (size_t)c, (size_t)j->T, (size_t)j->N, S);
        ofo_softmax(j->fwd, j->post, (size_t)c, (size_t)j->T, S);
    }
    return NULL;
}

static void *beam_worker(void *p) {
    job_t *j = (job_t *)p;
    const size_t S = (size_t)1 << (2 * j->state_len);
    const size_t T = (size_t)j->T;
    for (int c = j->first; c < j->last; ++c) {
        const size_t n = (size_t)c;
        int32_t *st = j->states + n * T;
        uint8_t *mv = j->moves + n * T;
        float *ql = j->qual + n * T * 4;
        float *bp = j->base_probs + n * T;
        float *tp = j->total_probs + n * T;
        ofo_beam_search(j->scores + n * 4 * S, (size_t)j->N * (size_t)j->C,
                        j->bwd_in + n * (T + 1) * S, j->post_in + n * (T + 1) * S,
                        2 * j->state_len, T, j->opt->beam_cut, j->opt->blank_score,
                        st, mv, ql, j->beam + n * OFO_BEAM_WIDTH * (T + 1),
                        j->path_states ? j->path_states + n * T : NULL);
        size_t seq_len = 0;
        for (size_t t = 0; t < T; ++t) { seq_len += mv[t]; bp[t] = 0.0f; tp[t] = 0.0f; }
        ofo_generate_sequence(mv, st, ql, j->opt->q_shift, j->opt->q_scale, T, seq_len, bp, tp,
                              j->sequence + n * T, j->qstring + n * T);
    }
    return NULL;
}

static void run_phase(void *(*fn)(void *), job_t *jobs, int nthreads) {
    pthread_t *tid = (pthread_t *)malloc(sizeof(pthread_t) * (size_t)nthreads);
    for (int t = 0; t < nthreads; ++t) if (pthread_create(&tid[t], NULL, fn, &jobs[t]) != 0) abort();
    for (int t = 0; t < nthreads; ++t) if (pthread_join(tid[t], NULL) != 0) abort();
    free(tid);
}

static void *pick(void *user, size_t bytes, void **owned) {
    if (user) { *owned = NULL; return user; }
    *owned = malloc(bytes);
    if (!*owned) abort();
    return *owned;
}

static void decode_impl(int T, int N, int C, int nthreads, const float *scores, int state_len,
                        const ofo_opt_t *opt, const float *bwd_in, const float *post_in,
                        uint8_t *moves, char *sequence, char *qstring, const ofo_dump_t *dump) {
    static const ofo_dump_t none = {0};
    if (!dump) dump = &none;
    const size_t S = (size_t)1 << (2 * state_len);
    const size_t NT = (size_t)N * (size_t)T;
    const size_t tens = (size_t)N * (size_t)(T + 1) * S;
    void *own[9] = {0};

    float *bwd = NULL, *fwd = NULL, *post = NULL;
    if (!bwd_in) {
        bwd = (float *)pick(dump->bwd, tens * sizeof(float), &own[0]);
        fwd = (float *)pick(dump->fwd, tens * sizeof(float), &own[1]);
        post = (float *)pick(dump->post, tens * sizeof(float), &own[2]);
    }
    int32_t *states = (int32_t *)pick(dump->states, NT * sizeof(int32_t), &own[3]);
    float *qual = (float *)pick(dump->qual_data, NT * 4 * sizeof(float), &own[4]);
    float *bp = (float *)pick(dump->base_probs, NT * sizeof(float), &own[5]);
    float *tp = (float *)pick(dump->total_probs, NT * sizeof(float), &own[6]);
    ofo_beam_slot_t *beam = (ofo_beam_slot_t *)pick(dump->beam, (size_t)N * OFO_BEAM_WIDTH * (size_t)(T + 1) * sizeof(ofo_beam_slot_t), &own[7]);

    memset(moves, 0, NT);
    memset(sequence, 0, NT);
    memset(qstring, 0, NT);

    if (nthreads > N) nthreads = N;
    if (nthreads < 1) nthreads = 1;
    const int share = N / nthreads, extra = N % nthreads;
    job_t *jobs = (job_t *)calloc((size_t)nthreads, sizeof(job_t));
    for (int t = 0; t < nthreads; ++t) {
        job_t *j = &jobs[t];
        j->first = t * share + (t < extra ? t : extra);
        j->last = j->first + share + (t < extra ? 1 : 0);
        j->T = T; j->N = N; j->C = C; j->state_len = state_len;
        j->scores = scores; j->opt = opt;
        j->bwd = bwd; j->fwd = fwd; j->post = post;
        j->bwd_in = bwd_in ? bwd_in : bwd;
        j->post_in = post_in ? post_in : post;
        j->states = states; j->path_states = dump->path_states; j->moves = moves; j->qual = qual;
        j->base_probs = bp; j->total_probs = tp;
        j->sequence = sequence; j->qstring = qstring; j->beam = beam;
    }
    if (!bwd_in) run_phase(scan_worker, jobs, nthreads);
    run_phase(beam_worker, jobs, nthreads);
    free(jobs);
    for (int i = 0; i < 9; ++i) free(own[i]);
}

void ofo_decode(int T, int N, int C, int nthreads, const float *scores, int state_len,
                const ofo_opt_t *opt, uint8_t *moves, char *sequence, char *qstring,
                const ofo_dump_t *dump) {
    decode_impl(T, N, C, nthreads, scores, state_len, opt, NULL, NULL, moves, sequence, qstring, dump);
}

void ofo_decode_from_tensors(int T, int N, int C, int nthreads, const float *scores, int state_len,
                             const ofo_opt_t *opt, const float *bwd, const float *post,
                             uint8_t *moves, char *sequence, char *qstring, const ofo_dump_t *dump) {
    decode_impl(T, N, C, nthreads, scores, state_len, opt, bwd, post, moves, sequence, qstring, dump);
}

/* ---- rotary embedding (src/nn_cpu.c:10-39, :80-132) ---------------------- */

typedef struct {
    float *x;
    const float *sn, *cs;
    int first, last, seqlen, nheads, half, sb, ss, sh;
} rot_job_t;

static void *rot_worker(void *p) {
    rot_job_t *j = (rot_job_t *)p;
    for (int b = j->first; b < j->last; ++b)
        for (int h = 0; h < j->nheads; ++h)
            for (int r = 0; r < j->half; ++r) {
                float *lo = j->x + (size_t)b * (size_t)j->sb + (size_t)h * (size_t)j->sh + (size_t)r;
                float *hi = lo + j->half;
                for (int s = 0; s < j->seqlen; ++s) {
                    const float c = j->cs[(size_t)s * (size_t)j->half + (size_t)r];
                    const float sn = j->sn[(size_t)s * (size_t)j->half + (size_t)r];
                    float *a = lo + (size_t)s * (size_t)j->ss, *d = hi + (size_t)s * (size_t)j->ss;
                    const float x0 = *a, x1 = *d;
                    *a = x0 * c - x1 * sn;
                    *d = x0 * sn + x1 * c;
                }
            }
    return NULL;
}

void ofo_rotary_emb(float *x, const float *sin_buf, const float *cos_buf, int batch, int seqlen,
                    int nheads, int head_dim, int rotary_half, int stride_batch, int stride_seq,
                    int stride_head, int nthreads) {
    (void)head_dim;
    if (nthreads > batch) nthreads = batch;
    if (nthreads < 1) nthreads = 1;
    const int share = batch / nthreads, extra = batch % nthreads;
    rot_job_t *jobs = (rot_job_t *)calloc((size_t)nthreads, sizeof(rot_job_t));
    pthread_t *tid = (pthread_t *)malloc(sizeof(pthread_t) * (size_t)nthreads);
    for (int t = 0; t < nthreads; ++t) {
        rot_job_t *j = &jobs[t];
        j->x = x; j->sn = sin_buf; j->cs = cos_buf;
        j->first = t * share + (t < extra ? t : extra);
        j->last = j->first + share + (t < extra ? 1 : 0);
        j->seqlen = seqlen; j->nheads = nheads; j->half = rotary_half;
        j->sb = stride_batch; j->ss = stride_seq; j->sh = stride_head;
        if (pthread_create(&tid[t], NULL, rot_worker, j) != 0) abort();
    }
    for (int t = 0; t < nthreads; ++t) pthread_join(tid[t], NULL);
    free(tid);
    free(jobs);
}
