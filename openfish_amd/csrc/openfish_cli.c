/*
 * Command-line driver: decode a score blob on the GPU and write the three result blobs,
 * the job the reference's test driver does (reference src/main.c:200-355, used by
 * test/test.sh:26-40).
 *
 *   openfish <scores.blob> <BATCH_SIZE> <STATE_LEN> [T]
 *
 * The blob holds T*N*C scores, TNC, C = 4*4^STATE_LEN (or 5*4^STATE_LEN), either as
 * fp16 (what the reference's GPU build reads) or as fp32 (what its CPU build reads; the
 * values are converted to fp16 on the host); the size of the file tells which.  T is
 * 1666 unless given.  Writes moves.blob, sequence.blob and qstring.blob (N*T bytes
 * each) into the current directory; with OPENFISH_DUMP_TENSORS=1 also the device
 * tensors (bwd_NTC, post_NTC, qual_data, base_probs, total_probs).
 *
 * OPENFISH_BENCH_BATCHES=<n> decodes the batch n times and reports the time of all of them, the
 * job of the reference driver's BENCH build (src/main.c:274-298; built with -DBENCH this driver takes
 * the reference's counts, 1400 / 3450 / 6850 batches for state_len 3 / 4 / 5, 140 otherwise, unless
 * the variable says otherwise).  The files hold the last batch's results.
 */
#include <errno.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

#include <openfish/openfish.h>
#include <openfish/openfish_amd.h>

static void fail(const char *what, const char *name) {
    fprintf(stderr, "openfish: %s %s: %s\n", what, name, strerror(errno));
    exit(EXIT_FAILURE);
}

/* IEEE fp32 -> fp16, round to nearest even */
static uint16_t to_half(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    const uint32_t sign = (x >> 16) & 0x8000u;
    const uint32_t mag = x & 0x7fffffffu;
    if (mag >= 0x7f800000u) return (uint16_t)(sign | 0x7c00u | (mag > 0x7f800000u ? 0x200u : 0));
    if (mag >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u); /* rounds to infinity */
    if (mag < 0x33000001u) return (uint16_t)sign;               /* rounds to zero */
    int exp = (int)(mag >> 23) - 127;
    uint32_t man = (mag & 0x7fffffu) | 0x800000u;
    int shift = exp < -14 ? 13 + (-14 - exp) : 13; /* subnormal halves lose more bits */
    uint32_t half_man = man >> shift;
    const uint32_t rest = man & ((1u << shift) - 1), mid = 1u << (shift - 1);
    if (rest > mid || (rest == mid && (half_man & 1u))) ++half_man;
    if (exp < -14) return (uint16_t)(sign | half_man); /* carry into the exponent is correct */
    return (uint16_t)(sign + ((uint32_t)(exp + 15) << 10) + (half_man - 0x400u));
}

static void write_blob(const char *name, const void *data, size_t bytes) {
    FILE *fp = fopen(name, "w");
    if (!fp) fail("cannot open", name);
    if (fwrite(data, 1, bytes, fp) != bytes) fail("error writing", name);
    fclose(fp);
}

int main(int argc, char *argv[]) {
    if (argc < 4) {
        fprintf(stderr, "Usage: %s <scores.blob> <BATCH_SIZE> <STATE_LEN> [T]\n", argv[0]);
        return EXIT_FAILURE;
    }
    set_openfish_log_level(OPENFISH_LOG_DBUG);
    const int N = (int)strtol(argv[2], NULL, 10);
    const int state_len = (int)strtol(argv[3], NULL, 10);
    const int T = argc > 4 ? (int)strtol(argv[4], NULL, 10) : 1666;
    if (N < 1 || T < 1 || state_len < 3 || state_len > 5) {
        fprintf(stderr, "openfish: need BATCH_SIZE >= 1, T >= 1 and STATE_LEN 3, 4 or 5\n");
        return EXIT_FAILURE;
    }
    const size_t S = (size_t)1 << (2 * state_len);

    FILE *fp = fopen(argv[1], "rb");
    if (!fp) fail("cannot open", argv[1]);
    if (fseek(fp, 0, SEEK_END) != 0) fail("cannot seek", argv[1]);
    const size_t bytes = (size_t)ftell(fp);
    rewind(fp);
    const size_t per4 = (size_t)T * (size_t)N * 4 * S, per5 = (size_t)T * (size_t)N * 5 * S;
    int C, elem;
    if (bytes == per4 * 2) { C = (int)(4 * S); elem = 2; }
    else if (bytes == per4 * 4) { C = (int)(4 * S); elem = 4; }
    else if (bytes == per5 * 2) { C = (int)(5 * S); elem = 2; }
    else if (bytes == per5 * 4) { C = (int)(5 * S); elem = 4; }
    else {
        fprintf(stderr, "openfish: %s has %zu bytes; expected T*N*C scores of 2 or 4 bytes with C = %zu or %zu\n",
                argv[1], bytes, 4 * S, 5 * S);
        return EXIT_FAILURE;
    }
    void *raw = malloc(bytes);
    if (!raw) fail("out of memory reading", argv[1]);
    if (fread(raw, 1, bytes, fp) != bytes) fail("error reading", argv[1]);
    fclose(fp);
    const size_t count = bytes / (size_t)elem;
    uint16_t *half = (uint16_t *)raw;
    if (elem == 4) {
        half = (uint16_t *)malloc(count * 2);
        if (!half) fail("out of memory converting", argv[1]);
        for (size_t i = 0; i < count; ++i) half[i] = to_half(((const float *)raw)[i]);
        free(raw);
    }

    set_device_hip(0);
    void *scores_gpu = upload_scores_to_hip(T, N, C, half);
    openfish_gpubuf_t *gpubuf = openfish_gpubuf_init(T, N, state_len);
    openfish_opt_t options = DECODER_INIT;
    /* per-model quality calibration as in the reference driver (src/main.c:253-265) */
    if (state_len == 3) { options.q_scale = 0.97f; options.q_shift = -1.8f; }
    else if (state_len == 4) { options.q_scale = 0.95f; options.q_shift = -0.2f; }
    else { options.q_scale = 0.95f; options.q_shift = 0.5f; }

    long n_batch = 1;
#ifdef BENCH
    n_batch = state_len == 3 ? 1400 : state_len == 4 ? 3450 : state_len == 5 ? 6850 : 140;
#endif
    const char *batches = getenv("OPENFISH_BENCH_BATCHES");
    if (batches && atol(batches) > 0) n_batch = atol(batches);

    uint8_t *moves = NULL;
    char *sequence = NULL, *qstring = NULL;
    struct timespec t0, t1;
    clock_gettime(CLOCK_MONOTONIC, &t0);
    for (long i = 0; i < n_batch; ++i) {
        if (i) {
            free(moves);
            free(sequence);
            free(qstring);
        }
        openfish_decode_gpu(T, N, C, scores_gpu, state_len, &options, gpubuf, &moves, &sequence, &qstring);
    }
    clock_gettime(CLOCK_MONOTONIC, &t1);
    const double secs = (double)(t1.tv_sec - t0.tv_sec) + 1e-9 * (double)(t1.tv_nsec - t0.tv_nsec);
    OPENFISH_LOG_DEBUG("decode completed in %f secs", secs);
    if (n_batch > 1)
        fprintf(stderr, "openfish: %ld batches of %d chunks in %f secs (%.0f chunks/s)\n", n_batch, N, secs,
                (double)n_batch * N / secs);

    const size_t nt = (size_t)N * (size_t)T;
    write_blob("moves.blob", moves, nt);
    write_blob("sequence.blob", sequence, nt);
    write_blob("qstring.blob", qstring, nt);
    const char *dump = getenv("OPENFISH_DUMP_TENSORS");
    if (dump && dump[0] == '1') write_gpubuf_hip((uint64_t)T, (uint64_t)N, state_len, gpubuf);

    free(moves);
    free(sequence);
    free(qstring);
    free(half);
    openfish_gpubuf_free(gpubuf);
    free_scores_hip(scores_gpu);
    return 0;
}
