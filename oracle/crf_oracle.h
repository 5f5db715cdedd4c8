/*
 * CPU oracle for the CRF-CTC decode path and the rotary embedding.
 *
 * TEST INFRASTRUCTURE ONLY.  This is a plain-C restatement of the reference
 * CPU algorithm (reference files src/decode_cpu.c, src/beam_search.c,
 * src/nn_cpu.c).  It exists to check the HIP kernels and to be timed as the
 * CPU baseline.  Nothing in the shipped library links, loads or calls it.
 *
 * Pinning status of each function (what independent evidence fixes it):
 *   ofo_backward_scan / ofo_forward_scan / ofo_softmax
 *       pinned: bit-for-bit against the compiled reference (oracle/_ref) on
 *       seeded inputs; closed form for constant scores; brute-force path
 *       enumeration for state_len 1; row sums of the posterior.
 *       With ofo_set_scan_stay at a value other than the reference CPU path's literal 2.0 (the
 *       reference's GPU scans take options->blank_score there, src/decode_hip.hip:120) no
 *       reference vector exists; that setting is pinned by the closed form
 *       (T-t) log(e^stay + 4 e^c) on constant scores and by dense transition-matrix products
 *       with e^stay on the diagonal (tests/test_oracle.py).
 *   ofo_crc32c            pinned: CRC-32C check value 0xE3069283 of "123456789".
 *   ofo_kth_largest       pinned: equals sort(desc)[k] on random and tied input.
 *   ofo_log_sum_exp       pinned: log(e^x+e^y) closed form, 17.0 cut-off.
 *   ofo_beam_search / ofo_generate_sequence / ofo_decode
 *       pinned: the reference's own golden vector (the blobs under test/data) and
 *       bit-for-bit against the compiled reference on seeded inputs for
 *       state_len 1..5, including a sharply peaked / near-uniform mix.
 *   ofo_rotary_emb        pinned: 2-D rotation closed form and the compiled
 *       reference.
 */
#ifndef CRF_ORACLE_H
#define CRF_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum {
    OFO_BASES = 4,
    OFO_BEAM_WIDTH = 32,
    OFO_MAX_STATES = 1024,
    OFO_MAX_CANDIDATES = 5 * OFO_BEAM_WIDTH
};

/* one persisted beam slot (reference: beam_element_t, src/decode.h:14-18) */
typedef struct {
    int32_t state;
    uint8_t prev;
    uint8_t stay;
} ofo_beam_slot_t;

/* decode options actually read by the reference (include/openfish/openfish.h:29-37) */
typedef struct {
    float beam_cut;
    float blank_score;
    float q_shift;
    float q_scale;
} ofo_opt_t;

/* optional intermediate tensors; any pointer may be NULL */
typedef struct {
    float *bwd;         /* [N][T+1][S] */
    float *fwd;         /* [N][T+1][S]  (holds fwd+bwd, as the reference does) */
    float *post;        /* [N][T+1][S] */
    int32_t *states;    /* [N][T]  (after the qual stage: state & 3) */
    int32_t *path_states; /* [N][T]  full k-mer state of the traced path */
    float *qual_data;   /* [N][T][4] */
    float *base_probs;  /* [N][T] */
    float *total_probs; /* [N][T] */
    ofo_beam_slot_t *beam; /* [N][T+1][32] */
} ofo_dump_t;

uint32_t ofo_crc32c(uint32_t crc, uint32_t bits, int nbits);
float ofo_kth_largest(float *v, int k, int n);
float ofo_log_sum_exp(float x, float y);

/* test knob: the stay score the scans add (default: the reference CPU path's literal 2.0f).  Process-wide. */
void ofo_set_scan_stay(float stay);

/* scans over one chunk; scores is the fp32 [T][N][4S] tensor */
void ofo_backward_scan(const float *scores, float *bwd, size_t chunk, size_t T, size_t N, size_t S);
void ofo_forward_scan(const float *scores, const float *bwd, float *fwd, size_t chunk, size_t T, size_t N, size_t S);
void ofo_softmax(const float *fwd, float *post, size_t chunk, size_t T, size_t S);

/* beam search + traceback + per-block quality of one chunk.
 * scores points at the chunk's row 0; row_stride is the distance between rows.
 * bwd/post are that chunk's [T+1][S] tensors.  path_states may be NULL. */
void ofo_beam_search(const float *scores, size_t row_stride, const float *bwd, const float *post,
                     int state_bits, size_t T, float beam_cut, float stay_score,
                     int32_t *states, uint8_t *moves, float *qual_data,
                     ofo_beam_slot_t *beam, int32_t *path_states);

void ofo_generate_sequence(const uint8_t *moves, const int32_t *states, const float *qual_data,
                           float shift, float scale, size_t T, size_t seq_len,
                           float *base_probs, float *total_probs, char *sequence, char *qstring);

/* whole decode, mirrors openfish_decode_cpu; outputs are caller-provided [N][T] buffers (zeroed here) */
void ofo_decode(int T, int N, int C, int nthreads, const float *scores, int state_len,
                const ofo_opt_t *opt, uint8_t *moves, char *sequence, char *qstring,
                const ofo_dump_t *dump);

/* beam + sequence stage only, fed external bwd/post ([N][T+1][S]) */
void ofo_decode_from_tensors(int T, int N, int C, int nthreads, const float *scores, int state_len,
                             const ofo_opt_t *opt, const float *bwd, const float *post,
                             uint8_t *moves, char *sequence, char *qstring, const ofo_dump_t *dump);

void ofo_rotary_emb(float *x, const float *sin_buf, const float *cos_buf, int batch, int seqlen,
                    int nheads, int head_dim, int rotary_half, int stride_batch, int stride_seq,
                    int stride_head, int nthreads);

#ifdef __cplusplus
}
#endif
#endif
