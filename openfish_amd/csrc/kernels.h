/*
 * Launchers of the gfx950 kernels, callable from C.  Each returns 0 on success,
 * a hipError_t value if the launch failed, or OFK_BAD_ARGS if the arguments do
 * not fit what the kernel assumes (nothing is launched in that case).
 */
#ifndef OPENFISH_AMD_KERNELS_H
#define OPENFISH_AMD_KERNELS_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* longest chunk in time steps: the sequence stage keeps 14 bytes per step in LDS (160 KB) */
#define OFK_MAX_T 8192
#define OFK_BAD_ARGS (-1)
#define OFK_TOO_LARGE (-2)
#define OFK_BEAM_WIDTH 32

/* one persisted beam slot, 16 bit: state[9:0] | prev[14:10] | stay[15] */
typedef uint16_t ofk_beam_slot_t;

/* Arithmetic of the scan update max + log(sum exp):
 *   OFK_SCAN_TWO_TIER  hardware fp32 exp/log where its rounded result is provably the CPU path's,
 *                      the CPU path's double exp/log and fp32 roundings elsewhere (same results
 *                      as OFK_SCAN_PRECISE);
 *   OFK_SCAN_PRECISE   the CPU path's double exp/log and fp32 roundings everywhere;
 *   OFK_SCAN_FAST      hardware fp32 exp/log everywhere (last-bit differences).
 * spl: states per lane, 4, 2 or 1; 0 chooses from the batch size.
 * columns: fp16 values per state in scores, 4 (the transitions) or 5 (an unused blank, then the
 * transitions); five-column scores are read where they lie. */
#define OFK_SCAN_TWO_TIER 0
#define OFK_SCAN_PRECISE 1
#define OFK_SCAN_FAST 2
int ofk_bwd_scan(const void *scores, float *bwd, int T, int N, int state_len, int columns, float stay, int mode,
                 int spl, void *stream);
int ofk_fwd_post_scan(const void *scores, const float *bwd, float *post, int T, int N, int state_len,
                      int columns, float stay, int mode, int spl, void *stream);
/* Both sweeps and the posterior in one kernel: the forward and backward recursions of a chunk run
 * side by side in one workgroup and meet in the middle of the chunk (same tensors as
 * ofk_bwd_scan followed by ofk_fwd_post_scan).  Rows 0 .. T/2-1 of post hold forward values
 * while the kernel runs. */
int ofk_scan_posterior(const void *scores, float *bwd, float *post, int T, int N, int state_len,
                       int columns, float stay, int mode, int spl, void *stream);
/* Table behind log(1 + e^-gap), the correction of a pairwise log-sum-exp, for gap in
 * [0, 17): OFK_LSE_CELLS cells of width 1/4, each a degree-8 polynomial in
 * s = 8 * (gap - centre) in [-1, 1], coefficients lowest degree first.  Built on the
 * host in long double (ofk_lse_table_build), absolute error below 2^-46. */
#define OFK_LSE_CELLS 68
#define OFK_LSE_COEFS 9
#define OFK_LSE_DOUBLES (OFK_LSE_CELLS * OFK_LSE_COEFS)

int ofk_beam_search(const void *scores, const float *bwd, ofk_beam_slot_t *beam, int32_t *states,
                    uint8_t *moves, int T, int N, int state_len, int columns, float log_beam_cut, float stay,
                    const double *lse_table, int flags, void *stream);
/* The same search with the beam slots and the table in a static device array of the library
 * (OFK_STATIC_SLOT_BYTES of slots: N * (T + 1) * 64 bytes must fit, else OFK_TOO_LARGE and nothing
 * is launched).  ofk_beam_search_static_prepare sets the array up on the current device (looks up
 * its address, copies the 612 doubles at lse_table_host, host memory, into it with a blocking
 * copy; a no-op once done).  ofk_beam_search_static then only launches the kernel on `stream`: it
 * allocates nothing, copies nothing and waits for nothing (OFK_NOT_PREPARED if the device's array
 * has not been set up).  Calls that overlap in time on one device share the array and race. */
#define OFK_STATIC_SLOT_BYTES (64u << 20)
#define OFK_NOT_PREPARED (-3)
int ofk_beam_search_static_prepare(const double *lse_table_host);
int ofk_beam_search_static_ready(void);
int ofk_beam_search_static(const void *scores, const float *bwd, int32_t *states, uint8_t *moves, int T, int N,
                           int state_len, int columns, float log_beam_cut, float stay, int flags, void *stream);
/* flags, for tests.  Bit 0: replay every stay/step merge one by one in CPU order (the path
 * otherwise taken only after a hash collision); results must not change.  Bit 1: seed hashes are
 * taken from (state & 15), so that different sequences share hashes and the search has to notice
 * the duplicates by itself; results then equal those of a CPU search seeded the same way. */
/* Phred characters run from '"' (34, q = 1) to 'S' (83, q = 50).  thr[j] is the smallest
 * miss probability x whose character is at most 82 - j (2.0f if no x in [0,1] reaches it),
 * so that char(x) = 83 - #{j : x >= thr[j]}. */
#define OFK_PHRED_STEPS 49
typedef struct {
    float thr[OFK_PHRED_STEPS];
} ofk_phred_table_t;

/* path_sums: NULL, or what ofk_path_sums left for these posteriors (post is then not read). */
int ofk_sequence(const float *post, int32_t *states, const uint8_t *moves, float *qual_data,
                 float *base_probs, float *total_probs, char *sequence, char *qstring, int T, int N,
                 int state_len, const ofk_phred_table_t *phred, const float *path_sums, void *stream);
/* sums[n][t][s], N x T x states floats: posterior of state s at row t + 1 of chunk n plus that of its
 * distinct one-base shifts, fp32 sums in the CPU path's order (src/beam_search.c:441-463), for every
 * state: the input of a block's quality whichever state the path then takes. */
int ofk_path_sums(const float *post, float *sums, int T, int N, int state_len, void *stream);
/* Batches up to this size put at most two chunks of the beam search on a compute unit (one wave
 * each): the search then leaves room for ofk_path_sums beside it.  Larger batches fill the units
 * with search waves, and the extra kernel was measured to cost the search more than it saves the
 * sequence stage (1024 chunks of 256 states: search 1.42 -> 1.77 ms, sequence 0.32 -> 0.13 ms). */
#define OFK_SPARSE_SEARCH_MAX_CHUNKS 512
/* device-to-device copy of `bytes` (a multiple of 16); the calibration kernel for counters */
int ofk_copy(void *dst, const void *src, size_t bytes, void *stream);
int ofk_rotary_emb(void *x, const float *sin_buf, const float *cos_buf, int batch, int seqlen,
                   int nheads, int rotary_half, long stride_batch, long stride_seq, long stride_head,
                   void *stream);

/* Worst errors of v_exp_f32 over every fp32 in [-160, 0] (relative, results in the normal range)
 * and of v_log_f32 over every fp32 in [1, 2), [2, 4), [4, 5.01] (absolute), against double
 * arithmetic, plus the identities exp2(0) = exp2(-0) = 1, log2(1) = 0, log2(2) = 1.  The results
 * go to 40 bytes of device memory at scratch40 (8-byte aligned): four doubles, then a word of
 * identity bits (bit 0..3 in the order above). */
int ofk_probe_hw_math(void *scratch40, void *stream);

#ifdef __cplusplus
}
#endif
#endif
