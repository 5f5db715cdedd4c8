/*
 * Public C API of the MI355X-native openfish CRF-CTC decoder.
 *
 * Names, argument order, struct layouts and ownership rules are those of the
 * reference header (reference include/openfish/openfish.h:14-102) so that a
 * caller built against the reference links against this library unchanged.
 * There is one backend here (HIP, gfx950); nothing is selected at compile time.
 */
#ifndef OPENFISH_H
#define OPENFISH_H

#include <stdbool.h>
#include <stdint.h>
#include <stdlib.h>

#include "openfish_error.h"

#ifdef __cplusplus
extern "C" {
#endif

/* beam_width, beam_cut, blank_score, q_shift, q_scale, temperature, move_pad */
#define DECODER_INIT {32, 100.0, 2.0, 0.0, 1.0, 1.0, false}

/*
 * Decode options (reference openfish.h:29-37).  As in the reference only
 * beam_cut, blank_score, q_shift and q_scale are read; the beam is 32 wide.
 */
typedef struct openfish_opt {
    size_t beam_width;
    float beam_cut;
    float blank_score;
    float q_shift;
    float q_scale;
    float temperature;
    bool move_pad;
} openfish_opt_t;

/*
 * Device scratch of one decoder instance (reference openfish.h:16-27), created
 * by openfish_gpubuf_init for a maximum batch shape and reused across calls.
 * bwd_NTC and post_NTC are fp32 [N][T+1][4^state_len]; moves, sequence and
 * qstring are [N][T] bytes; qual_data is fp32 [N][T][4]; base_probs and
 * total_probs are fp32 [N][T]; states is int32 [N][T].  beam_vector is private
 * to the library.
 */
typedef struct openfish_gpubuf {
    float *bwd_NTC;
    float *post_NTC;
    uint8_t *moves;
    char *sequence;
    char *qstring;
    void *beam_vector;
    void *states;
    float *qual_data;
    float *base_probs;
    float *total_probs;
} openfish_gpubuf_t;

/* reference src/decode_hip.hip:13-51 (ten device allocations sized from T, N, state_len) */
openfish_gpubuf_t *openfish_gpubuf_init(const int T, const int N, const int state_len);

/* reference src/decode_hip.hip:53-81 */
void openfish_gpubuf_free(openfish_gpubuf_t *gpubuf);

/*
 * Decode a batch on the current device (reference src/openfish.c:43-63,
 * src/decode_hip.hip:83-217).
 *   scores_TNC  device pointer, T*N*C IEEE half, TNC contiguous, C = 4*4^state_len
 *               (the reference's layout: element 4*state + dropped base).  C = 5*4^state_len
 *               is also accepted: element 5*state is then a blank column that is skipped
 *               and elements 5*state + 1 + base are the four step scores.
 *   *moves, *sequence, *qstring
 *               on return host buffers of N*T bytes each obtained with malloc;
 *               chunk n starts at n*T; sequence/qstring hold seq_len characters
 *               followed by zeros.  The caller frees them.
 * The call is synchronous.  Any failure prints to stderr and exits.
 */
void openfish_decode_gpu(const int T, const int N, const int C, void *scores_TNC,
                         const int state_len, const openfish_opt_t *options,
                         const openfish_gpubuf_t *gpubuf, uint8_t **moves, char **sequence,
                         char **qstring);

/*
 * In-place rotary embedding on the current device (reference src/openfish.c:65-110,
 * src/nn_hip.hip:11-43, src/rotary_emb_hip.h:36-70).  x_gpu is half, sin_gpu and
 * cos_gpu are fp32 [seqlen][rotary_half]; strides are in elements.  Synchronous.
 */
void openfish_rotary_emb_gpu(void *x_gpu, void *sin_gpu, void *cos_gpu, int batch_size, int seqlen,
                             int nheads, int head_dim, int rotary_half, int stride_batch,
                             int stride_seq, int stride_head);

/*
 * CPU entry points of the reference API (reference src/decode_cpu.c:231,
 * src/nn_cpu.c:80).  This library carries the GPU path only: both symbols exist
 * so that callers link, print an error and exit when called.
 */
void openfish_decode_cpu(const int T, const int N, const int C, int nthreads, void *scores_TNC,
                         const int state_len, const openfish_opt_t *options, uint8_t **moves,
                         char **sequence, char **qstring);
void openfish_rotary_emb_cpu(void *x, void *sin_buf, void *cos_buf, int batch_size, int seqlen,
                             int nheads, int head_dim, int rotary_half, int stride_batch,
                             int stride_seq, int stride_head, int nthreads);

#ifdef __cplusplus
}
#endif

#endif /* OPENFISH_H */
