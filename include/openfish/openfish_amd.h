/*
 * Stage-level C-ABI of the MI355X decoder: the same work openfish_decode_gpu
 * does, one stage at a time, on caller-provided device buffers.  Used by
 * parity tests and benchmarks; plain pointers and sizes only.
 *
 * Every function works on the current device, is synchronous unless stated,
 * and follows the library's error convention (message on stderr, exit).
 */
#ifndef OPENFISH_AMD_H
#define OPENFISH_AMD_H

#include <stddef.h>
#include <stdint.h>

#include "openfish.h"

#ifdef __cplusplus
extern "C" {
#endif

/* ---- device helpers (reference src/decode_hip.h:34-54, src/decode_hip.hip:220-346) ---- */

/* reference set_device_hip, src/decode_hip.hip:220-226 */
void set_device_hip(int device);
/* reference upload_scores_to_hip, src/decode_hip.hip:228-244: host half [T][N][C] -> new device buffer */
void *upload_scores_to_hip(const int T, const int N, const int C, const void *scores_TNC);
/* reference free_scores_hip, src/decode_hip.hip:246-252 */
void free_scores_hip(void *scores_TNC_gpu);
/* reference write_gpubuf_hip, src/decode_hip.hip:254-346: dumps bwd_NTC, post_NTC, qual_data,
 * base_probs, total_probs of a gpubuf as <name>.blob into the current directory */
void write_gpubuf_hip(const uint64_t T, const uint64_t N, const int state_len,
                      const openfish_gpubuf_t *gpubuf);

/* raw device memory for harnesses that have no HIP binding of their own */
void *openfish_amd_malloc(size_t bytes);
void openfish_amd_free(void *dev);
void openfish_amd_memcpy_h2d(void *dev, const void *host, size_t bytes);
void openfish_amd_memcpy_d2h(void *host, const void *dev, size_t bytes);
void openfish_amd_memset(void *dev, int value, size_t bytes);
void openfish_amd_sync(void);
/* device-to-device copy by a plain kernel (reads `bytes`, writes `bytes`; multiple of 16):
 * the kernel of known traffic against which hardware counters are calibrated */
void openfish_amd_copy(void *dst, const void *src, size_t bytes);
/* number of visible devices; 0 when there is none (never exits) */
int openfish_amd_device_count(void);

/* ---- stages ---- */

/*
 * Arithmetic of the scan update max + log(sum of five exponentials) (reference
 * src/decode_cpu.c:45-49,104-108: exp and log in double, the running sum and the result
 * rounded to fp32).
 *   OPENFISH_AMD_SCAN_TWO_TIER (default): the update is first evaluated with the hardware's
 *     fp32 exp/log; where that result could round to another fp32 number than the CPU path's
 *     (it lies within the error bound of a rounding boundary) the update is re-evaluated with
 *     double exp/log and the CPU path's roundings.  Same tensors as _PRECISE.
 *   OPENFISH_AMD_SCAN_PRECISE: double exp/log and the CPU path's roundings for every update.
 *   OPENFISH_AMD_SCAN_FAST: hardware fp32 exp/log only; bwd within 2 ulp.  A last-bit
 *     difference of a scan value of magnitude 4096..8192 is a 5e-4 relative difference of the
 *     posterior built from it, so this mode is outside the 1e-3 acceptance bar on a few
 *     posteriors per ten million.  For measurements.
 */
enum openfish_amd_scan_mode {
    OPENFISH_AMD_SCAN_TWO_TIER = 0,
    OPENFISH_AMD_SCAN_PRECISE = 1,
    OPENFISH_AMD_SCAN_FAST = 2
};

/*
 * Backward scan (reference backward_scan src/decode_cpu.c:13-52, GPU twin
 * bwd_scan src/scan_hip.hip:9-58).  scores: device half [T][N][C], C = 4*S, or 5*S with an
 * unused blank value in front of the four of every state (all stages take both layouts).
 * bwd: device fp32 [N][T+1][S], row T is zero.
 */
void openfish_amd_bwd_scan(int T, int N, int C, const void *scores, int state_len, float stay_score,
                           int scan_mode, float *bwd);

/*
 * Forward scan fused with the per-time-step posterior softmax (reference
 * forward_scan + softmax src/decode_cpu.c:54-147, GPU twin fwd_post_scan
 * src/scan_hip.hip:60-200).  post: device fp32 [N][T+1][S].
 */
void openfish_amd_fwd_post_scan(int T, int N, int C, const void *scores, int state_len,
                                float stay_score, int scan_mode, const float *bwd, float *post);

/*
 * Both scans and the posterior in one kernel (what openfish_decode_gpu runs by default): the
 * backward and the forward recursion of a chunk advance side by side and meet in the middle of
 * the chunk.  Same tensors as openfish_amd_bwd_scan followed by openfish_amd_fwd_post_scan.
 */
void openfish_amd_scan_posterior(int T, int N, int C, const void *scores, int state_len,
                                 float stay_score, int scan_mode, float *bwd, float *post);

/*
 * Beam search and traceback (reference beam_search_cpu src/beam_search.c:117-439).
 * Reads scores and bwd, fills gpubuf->beam_vector, gpubuf->states (int32 [N][T],
 * the full k-mer state of the traced path) and gpubuf->moves.
 */
void openfish_amd_beam_search(int T, int N, int C, const void *scores, int state_len,
                              const openfish_opt_t *options, const float *bwd,
                              const openfish_gpubuf_t *gpubuf);

/*
 * The same beam search and traceback for callers that must not allocate device memory while they
 * run (tight serving loops, harnesses that forbid it, code that records its launches on a stream):
 * it has no counterpart in the reference.  Instead of a gpubuf it uses a static array of the
 * library in device memory (64 MiB of beam slots plus the log-sum-exp table, held by every GPU the
 * library runs on until the process ends) and writes its results to caller-provided device
 * buffers: states int32 [N][T] (the k-mer state of the traced path) and moves uint8 [N][T].
 *
 * openfish_amd_beam_search_static_prepare() sets the array up on the current device, once: it looks
 * up the array's address and copies the 4.9 KB table into it with a blocking copy (not for use
 * inside a stream capture; later calls on the same device return at once).
 *
 * openfish_amd_beam_search_static(...) then only launches the kernel on `stream` (NULL: the null
 * stream) and returns without waiting: it calls no hipMalloc/hipFree, no copy and no
 * synchronisation; the results are valid once the stream has reached the launch.  It exits with a
 * message if the device has not been prepared, or if N * (T + 1) * 64 bytes exceed the 64 MiB (hac
 * at T = 1666: N <= 628).  All calls on one GPU share the array: calls that overlap in time race.
 */
void openfish_amd_beam_search_static_prepare(void);
void openfish_amd_beam_search_static(int T, int N, int C, const void *scores, int state_len,
                                     const openfish_opt_t *options, const float *bwd, int32_t *states,
                                     uint8_t *moves, void *stream);

/* free device memory in bytes (hipMemGetInfo): lets a test see that a call allocated nothing */
size_t openfish_amd_device_free_bytes(void);

/*
 * Per-block quality, base calls and phred string (reference src/beam_search.c:441-496
 * and generate_sequence_cpu src/beam_search.c:49-99).  Reads post, gpubuf->states and
 * gpubuf->moves; fills gpubuf->qual_data, base_probs, total_probs, sequence, qstring
 * and reduces gpubuf->states to the emitted base (state & 3) as the reference does.
 */
void openfish_amd_sequence(int T, int N, int state_len, const openfish_opt_t *options,
                           const float *post, const openfish_gpubuf_t *gpubuf);

/*
 * Beam search + sequence stage fed with external bwd/post tensors (device fp32
 * [N][T+1][S]); outputs as openfish_decode_gpu.  This is the entry the bit-exact
 * acceptance test uses with the CPU path's own tensors.
 */
void openfish_amd_decode_from_tensors(int T, int N, int C, const void *scores, int state_len,
                                      const openfish_opt_t *options, const float *bwd,
                                      const float *post, const openfish_gpubuf_t *gpubuf,
                                      uint8_t **moves, char **sequence, char **qstring);

/*
 * openfish_decode_gpu in two halves, for a caller that keeps more than one batch in
 * flight from one thread (one gpubuf per batch in flight).  The blocking call of the
 * reference (src/openfish.c:43-63, src/decode_hip.hip:83-217: five device
 * synchronisations and three host allocations per call) is enqueue + wait + a copy
 * into fresh malloc'd buffers.
 *
 * openfish_amd_decode_enqueue queues every kernel and the copies of the results into
 * the gpubuf's pinned host buffer, ordered after work already queued on the null
 * stream, and returns without waiting.  The scores must stay valid and unchanged until
 * the wait returns.  A gpubuf holds one enqueued decode at a time.
 *
 * openfish_amd_decode_wait blocks until that decode is complete and hands out pointers
 * into the pinned buffer: N*T bytes each, chunk n at n*T, as openfish_decode_gpu lays
 * them out.  They stay valid until the next enqueue (or decode) on the same gpubuf and
 * belong to the gpubuf: the caller does not free them.
 */
void openfish_amd_decode_enqueue(int T, int N, int C, const void *scores_TNC, int state_len,
                                 const openfish_opt_t *options, const openfish_gpubuf_t *gpubuf);
void openfish_amd_decode_wait(const openfish_gpubuf_t *gpubuf, const uint8_t **moves,
                              const char **sequence, const char **qstring);

/* ---- measurement ---- */

enum openfish_amd_stage {
    OPENFISH_AMD_STAGE_BWD = 0,   /* backward scan kernel (0 when both scans ran as one kernel) */
    OPENFISH_AMD_STAGE_FWD = 1,   /* forward + posterior kernel (0 when both scans ran as one kernel) */
    OPENFISH_AMD_STAGE_BEAM = 2,  /* beam search + traceback kernel */
    OPENFISH_AMD_STAGE_SEQ = 3,   /* quality + sequence kernel */
    OPENFISH_AMD_STAGE_TOTAL = 4, /* first launch to last kernel end, device side */
    OPENFISH_AMD_STAGE_SCAN = 5,  /* both scans + posterior as one kernel (0 when they ran split) */
    OPENFISH_AMD_STAGE_SUMS = 6,  /* per-state sums of posteriors for the quality stage, a kernel that runs beside the
                                   * beam search on a second stream (0 when the decode did without it) */
    OPENFISH_AMD_STAGE_COUNT = 7
};

/*
 * Device-side durations in milliseconds (HIP events on the streams the kernels
 * ran on) of the most recent openfish_decode_gpu call on this gpubuf.  Writes
 * min(n, OPENFISH_AMD_STAGE_COUNT) values and returns that count.
 */
int openfish_amd_last_timings(const openfish_gpubuf_t *gpubuf, float *ms, int n);

/*
 * Settings of one gpubuf, read whenever a decode (or a stage that takes the gpubuf) is queued
 * on it.  Nothing here is process-wide: two host threads with a gpubuf each do not see each
 * other's settings (the reference keeps no state beyond the log level either,
 * src/decode_hip.hip:83-217).  Not to be changed while a decode is enqueued on the gpubuf.
 *
 * scan mode: one of enum openfish_amd_scan_mode, default OPENFISH_AMD_SCAN_TWO_TIER.
 * states per lane: tuning knob of the scans, how many of the 4^state_len states one lane
 *   carries (4, 2 or 1); 0, the default, picks the largest value that still gives every SIMD of
 *   the device a wavefront for the batch at hand.  Results do not depend on it.
 * debug flags: bit 0 makes the beam search replay every stay/step merge serially in the CPU
 *   path's order, the route it otherwise takes only after a CRC collision between beam hashes;
 *   outputs must be identical with and without it.  Bit 1 seeds the beam with hashes of
 *   (state & 15) instead of the state, so that different sequences share hashes and that route
 *   is found by the search's own duplicate detection; for tests against a CPU search seeded
 *   the same way, never for real decoding.
 * split scans: 0 runs both scans and the posterior as one kernel, then the beam search; 1 runs the
 *   backward scan, then the forward scan + posterior on a second stream beside the beam search.
 *   Same results.  The first arrangement has the shorter scan stage at every batch size; the second
 *   hides the forward scan beneath the beam search, which pays while that search, one wavefront per
 *   chunk, leaves the machine idle.  A negative value, the default, lets every call choose: split
 *   for up to 512 chunks of 256 states (2048 of 64), one kernel beyond that and for 1024 states.
 */
void openfish_amd_gpubuf_set_scan_mode(const openfish_gpubuf_t *gpubuf, int scan_mode);
void openfish_amd_gpubuf_set_split_scans(const openfish_gpubuf_t *gpubuf, int split);
void openfish_amd_gpubuf_set_scan_states_per_lane(const openfish_gpubuf_t *gpubuf, int spl);
void openfish_amd_gpubuf_set_debug_flags(const openfish_gpubuf_t *gpubuf, int flags);

/*
 * The 49 miss-probability thresholds behind the phred characters for one
 * (q_scale, q_shift): char(x) = 83 - #{j : x >= thr[j]} equals
 * (char)(33.5f + clamp(-10*log10f(x)*q_scale + q_shift, 1, 50)) of the reference
 * (src/beam_search.c:92-97) for every x in [0,1].  Host-only; needs no device.
 */
void openfish_amd_phred_table(float q_scale, float q_shift, float *thr49);

/*
 * The table behind log(1 + e^-gap), gap in [0, 17), that the beam search uses when it
 * folds a stay into a step (reference log_sum_exp, src/beam_search.c:43-47): 68 cells of
 * width 1/4, each 9 coefficients (lowest degree first) of a polynomial in
 * s = 8 * (gap - cell centre).  Writes 612 doubles.  Host-only; needs no device.
 */
void openfish_amd_lse_table(double *out);

/*
 * Measures, on the current device, the worst error of the two hardware transcendentals the
 * default scan arithmetic and the beam search's merges build on, over every fp32 input of the
 * ranges they are used on, against double arithmetic; in units of 2^-24:
 *   errors4[0]  v_exp_f32, largest relative error over [-160, 0] (results in the normal range)
 *   errors4[1..3]  v_log_f32, largest absolute error over [1, 2), [2, 4), [4, 5.01]
 * identities: bit 0 exp2(0) == 1, bit 1 exp2(-0) == 1, bit 2 log2(1) == 0, bit 3 log2(2) == 1.
 * The two-tier evaluations are exact while these stay within 1.43, 1.0, 2.0, 4.0 and all four
 * identities hold (csrc/dmath.h, csrc/beam.hip); a test asserts that on the device at hand.
 * No counterpart in the reference, whose GPU path makes no claim of bit-exactness.
 */
void openfish_amd_probe_hw_math(double *errors4, unsigned int *identities);

/* library build tag, e.g. "openfish-amd gfx950" */
const char *openfish_amd_version(void);

#ifdef __cplusplus
}
#endif

#endif /* OPENFISH_AMD_H */
