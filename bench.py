#!/usr/bin/env python3
"""Throughput of the CRF-CTC decode on one MI355X, next to the CPU path.

One step = one `openfish_decode_gpu` call (backward scan, beam search, forward +
posterior scan, sequence stage, copy of moves/sequence/qstring to the host) over
one batch of synthetic scores that already sit in HBM.  The default workload is
the headline configuration: hac model (state_len 4, 256 states, C = 1024),
T = 1666, N = 512 chunks, fp16 scores drawn N(0, 2) (+1 on the dropped blank
column), beam width 32, beam cut 100, blank score 2.0.

Prints ONE JSON line:
  value      chunks decoded per second (wall clock around the K timed calls)
  roofline   the longest-running kernel: algorithmic bytes / mean device time
             (HIP events recorded by the library on the kernel's own stream)
  stages     every kernel's mean device time and algorithmic GB/s
  cpu_baseline  the CPU path timed on this host on a bounded sample of the same tensor
"""
import argparse
import json
import os
import statistics
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

WORKLOADS = {
    # name: (state_len, T, N, stress, q_scale, q_shift)
    "fast": (3, 1666, 512, False, 0.97, -1.8),
    "hac": (4, 1666, 512, False, 0.95, -0.2),
    "sup": (5, 1666, 256, False, 0.95, 0.5),
    "hac_stress": (4, 1666, 1024, True, 0.95, -0.2),
}
HBM_PEAK_GBS = 8000.0

TRAFFIC_FILE = os.path.join(ROOT, "profiles", "traffic.json")


def measured_traffic(workload, N, columns, kernel):
    """HBM bytes per launch of one kernel as rocprofv3 counted them (FETCH_SIZE + WRITE_SIZE, each
    scaled by the plain copy kernel's reading of the same counter): read from the summary the
    profiling script wrote (profiles/traffic.json); None where that run has not been made"""
    try:
        with open(TRAFFIC_FILE) as fh:
            table = json.load(fh)
    except (OSError, ValueError):
        return None
    entry = table.get("%s_n%d_c%d" % (workload, N, columns), {}).get(kernel)
    return None if entry is None else int(round(entry["hbm_bytes"]))


def algorithmic_bytes(state_len, T, N, columns=4):
    """bytes each kernel has to move at least once, per launch (C = columns * S scores per time step)"""
    S = 4 ** state_len
    C = columns * S
    scores = T * C * 2
    vec = (T + 1) * S * 4
    need = {
        "bwd": N * (scores + vec),                    # read scores, write bwd
        "fwd_post": N * (scores + 2 * vec),           # read scores + bwd, write post
        "beam": N * (scores + T * S * 4 + (T + 1) * 32 * 2 * 2 + 5 * T),  # rows, beam slots out+in, states+moves
        "sequence": N * (9 * 4 * T + 5 * T + 16 * T + 8 * T + 2 * T),  # gathers, states/moves, qual, probs, text
        "path_sums": N * 2 * T * S * 4,               # read the posteriors of T rows, write a sum per state
    }
    need["scan"] = need["bwd"] + need["fwd_post"]     # both scans + posterior as one kernel: the same minimum
    return need


def cpu_baseline(s16, state_len, opt_kw, sample_chunks):
    """the reference CPU path (oracle/_ref when it was built, else the oracle port) on the
    first `sample_chunks` chunks of the same tensor; median of 3 after one warm-up"""
    from oracle import crf_oracle as O
    T = s16.shape[0]
    sub = np.ascontiguousarray(s16[:, :sample_chunks, :]).astype(np.float32)
    cores = min(os.cpu_count() or 1, 16, sample_chunks)
    if O.have_ref():
        kind = "reference"
        run = lambda: O.ref_decode(sub, state_len, opt_kw, nthreads=cores)  # noqa: E731
    else:
        kind = "port"
        run = lambda: O.decode(sub, state_len, opt_kw, nthreads=cores, dump=False)  # noqa: E731
    run()
    times = []
    for _ in range(3):
        t0 = time.perf_counter()
        run()
        times.append(time.perf_counter() - t0)
    sec = statistics.median(times)
    return {"value": sample_chunks / sec, "unit": "chunks/s", "cores": cores, "kind": kind,
            "sample": "first %d chunks of the same tensor, T=%d, fp32 copy of the fp16 values, "
                      "median of 3 calls of openfish_decode_cpu (%.3f s each)" % (sample_chunks, T, sec)}


def cpu_baseline_config1(seed):
    """BASELINE's first configuration, the one the reference runs on the CPU: fast model (state_len 3,
    64 states), T=1666, N=16 chunks, fp32 scores (the fp16-rounded values of the generator), beam 32,
    beam cut 100, blank 2.0, q_shift 0, q_scale 1, on 8 threads, the thread count of the reference's
    own driver (src/main.c:287)"""
    from openfish_amd import synth
    from oracle import crf_oracle as O
    state_len, T, N, threads = 3, 1666, 16, 8
    s32 = synth.crf_scores(T, N, state_len, seed=seed, threads=8).astype(np.float32)
    opt_kw = dict(beam_cut=100.0, blank_score=2.0, q_shift=0.0, q_scale=1.0)
    if O.have_ref():
        kind = "reference"
        run = lambda: O.ref_decode(s32, state_len, opt_kw, nthreads=threads)  # noqa: E731
    else:
        kind = "port"
        run = lambda: O.decode(s32, state_len, opt_kw, nthreads=threads, dump=False)  # noqa: E731
    run()
    times = []
    for _ in range(5):
        t0 = time.perf_counter()
        run()
        times.append(time.perf_counter() - t0)
    sec = statistics.median(times)
    return {"value": round(N / sec, 1), "unit": "chunks/s", "cores": threads, "kind": kind,
            "sample": "fast: state_len 3, S=64, C=256 fp32, T=1666, N=16, beam 32, beam_cut 100, blank 2.0, q_shift 0, "
                      "q_scale 1; median of 5 calls of openfish_decode_cpu (%.4f s each)" % sec}


def rotary_bench(a):
    """in-place rotary embedding on the shape the reference's driver sketches
    (src/main.c:84-95): batch 500, seqlen 833, 8 heads of 64, rotary_half 32, half data"""
    from openfish_amd import api, synth
    batch, seqlen, nheads, head_dim, half = 500, 833, 8, 64, 32
    strides = (seqlen * nheads * head_dim, nheads * head_dim, head_dim)
    rng = np.random.default_rng(a.seed)
    x = rng.standard_normal((batch, seqlen, nheads, head_dim), dtype=np.float32).astype(np.float16)
    sn, cs = synth.rotary_tables(seqlen, half)
    xd, sd, cd = api.DeviceBuffer.from_host(x), api.DeviceBuffer.from_host(sn), api.DeviceBuffer.from_host(cs)
    call = lambda: api.openfish_rotary_emb_gpu(xd, sd, cd, batch, seqlen, nheads, head_dim, half, *strides)  # noqa: E731
    for _ in range(a.warmup):
        call()
    t0 = time.perf_counter()
    for _ in range(a.steps):
        call()
    ms = 1e3 * (time.perf_counter() - t0) / a.steps
    nbytes = 2 * x.nbytes + sn.nbytes + cs.nbytes  # x read and written once, tables read once
    gbs = nbytes / 1e9 / (ms / 1e3)
    print(json.dumps({
        "metric": "rotary embedding, in place, half", "value": round(gbs, 1), "unit": "GB/s", "n_gpus": 1,
        "steps": a.steps, "warmup": a.warmup, "ms_per_step": round(ms, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "rotary: batch 500, seqlen 833, 8 heads x 64, rotary_half 32 (half x, fp32 sin/cos); "
                               "time of the synchronous call, launch and sync included"},
        "roofline": {"bound": "hbm", "kernel": "rotary_vec8", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(gbs / HBM_PEAK_GBS, 4),
                     # measured: 0.426 GB written, 0.220 GB fetched -- about half of the tensor the
                     # previous call wrote is still in the 256 MB last-level cache
                     "traffic": 647000000},
        "cpu_baseline": None}))


def timed_decodes(api, gpubuf, call_args, steps):
    """`steps` blocking decodes: wall-clock ms per call and the mean device time of every stage"""
    per_stage = {k: [] for k in api.STAGES}
    api.lib().openfish_amd_sync()
    t0 = time.perf_counter()
    for _ in range(steps):
        api.openfish_decode_gpu_discard(*call_args, gpubuf)
        for k, v in gpubuf.timings().items():
            per_stage[k].append(v)
    api.lib().openfish_amd_sync()
    ms = 1e3 * (time.perf_counter() - t0) / steps
    return ms, {k: statistics.mean(v) for k, v in per_stage.items()}


def scan_stage(need, mean):
    """scans + posterior: one kernel (`scan`) or the two split kernels (`bwd`, `fwd_post`)"""
    ms = mean["scan"] + mean["bwd"] + mean["fwd_post"]
    gbs = need["scan"] / 1e9 / (ms / 1e3)
    return {"ms": round(ms, 4), "algorithmic_GB": round(need["scan"] / 1e9, 4), "GBps": round(gbs, 1),
            "frac_of_hbm_peak": round(gbs / HBM_PEAK_GBS, 4)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="hac", choices=sorted(WORKLOADS) + ["rotary"])
    ap.add_argument("--chunks", type=int, default=0, help="override N")
    ap.add_argument("--columns", type=int, default=4, choices=(4, 5),
                    help="scores per state and time step: 4 (what the reference consumes) or 5 (a blank column first, "
                         "C = 5 * 4^state_len as the network emits it)")
    ap.add_argument("--scan-mode", default="two_tier", choices=("two_tier", "precise", "fast"))
    ap.add_argument("--scans", default="auto", choices=("auto", "one", "split"),
                    help="arrangement of the scans: both as one kernel, or the backward scan and then the forward scan "
                         "beside the beam search; auto (the default): the library chooses per call")
    ap.add_argument("--split-scans", action="store_const", dest="scans", const="split", help="the same as --scans split")
    ap.add_argument("--states-per-lane", type=int, default=0, choices=(0, 1, 2, 4),
                    help="force the scans' states per lane (0: the library chooses)")
    ap.add_argument("--cpu-sample", type=int, default=512, help="chunks timed on the CPU path (0 = skip; capped at N)")
    ap.add_argument("--seed", type=int, default=20251125)
    ap.add_argument("--alt-steps", type=int, default=3,
                    help="extra timed calls per side measurement (split scans, hardware-exp scans), reported beside the "
                         "main result (0 = skip)")
    ap.add_argument("--no-five-columns", action="store_true",
                    help="skip the side measurement on the same scores with five columns per state (C = 5 * 4^state_len)")
    ap.add_argument("--overlap-steps", type=int, default=15,
                    help="calls per gpubuf of the two-batches-in-flight side measurement (0 = skip)")
    ap.add_argument("--copy-mib", type=int, default=1024,
                    help="size of the device copy whose GB/s is reported beside the 8 TB/s peak (0 = skip)")
    ap.add_argument("--calibrate-copy", type=int, default=0, metavar="MIB",
                    help="also run the plain copy kernel once over this many MiB (counter calibration)")
    a = ap.parse_args()
    if a.gpus != 1:
        sys.exit("bench.py: this decoder runs on one GPU; chunks are independent, so more GPUs means "
                 "one process and one batch shard per GPU (no collective). Run with --gpus 1.")

    from openfish_amd import api, synth
    if api.device_count() < 1:
        sys.exit("bench.py: no HIP device visible")

    if a.workload == "rotary":
        return rotary_bench(a)

    state_len, T, N, stress, q_scale, q_shift = WORKLOADS[a.workload]
    if a.chunks:
        N = a.chunks
    S = 4 ** state_len
    C = a.columns * S
    scale = synth.stress_scale(N) if stress else None
    five_side = a.columns == 4 and a.alt_steps > 0 and not a.no_five_columns
    made = synth.crf_scores(T, N, state_len, seed=a.seed, chunk_scale=scale, threads=16,
                            five_columns=a.columns == 5 or five_side)
    if a.columns == 5:
        s16, device_input, five = made[0], made[1], None  # s16: the four-column view
    elif five_side:
        s16, device_input, five = made[0], made[0], made[1]
    else:
        s16, device_input, five = made, made, None

    opt = api.DECODER_INIT(q_scale=q_scale, q_shift=q_shift)
    scores = api.upload_scores_to_hip(device_input)
    del made, device_input
    gpubuf = api.GpuBuf(T, N, state_len)
    gpubuf.set_scan_mode(a.scan_mode)
    asked = {"auto": None, "one": False, "split": True}[a.scans]
    gpubuf.set_split_scans(asked)
    gpubuf.set_scan_states_per_lane(a.states_per_lane)
    call = (T, N, C, scores, state_len, opt)

    if a.calibrate_copy:
        nbytes = a.calibrate_copy << 20
        src, dst = api.DeviceBuffer(nbytes), api.DeviceBuffer(nbytes)
        src.fill(1)
        api.lib().openfish_amd_copy(dst.ptr, src.ptr, nbytes)
        src.free()
        dst.free()

    for _ in range(a.warmup):
        api.openfish_decode_gpu_discard(*call, gpubuf)
    ms_per_step, mean = timed_decodes(api, gpubuf, call, a.steps)

    need = algorithmic_bytes(state_len, T, N, a.columns)
    stages = {}
    for k in ("scan", "bwd", "fwd_post", "beam", "sequence", "path_sums"):  # path_sums runs beside the beam search
        if mean[k] > 0:
            stages[k] = {"ms": round(mean[k], 4), "algorithmic_GB": round(need[k] / 1e9, 4),
                         "GBps": round(need[k] / 1e9 / (mean[k] / 1e3), 1)}
    stages["device_total_ms"] = round(mean["total"], 4)
    # kernels that share the machine: the beam search starts together with the forward scan (split scans) or
    # with the path sums (one scan kernel); their algorithmic bytes over the longer of the two
    beside = "fwd_post" if mean["fwd_post"] > 0 else ("path_sums" if mean["path_sums"] > 0 else None)
    if beside:
        window_ms = max(mean["beam"], mean[beside])
        gb = (need["beam"] + need[beside]) / 1e9
        stages["beam_and_" + beside + "_side_by_side"] = {
            "ms": round(window_ms, 4), "algorithmic_GB": round(gb, 4), "GBps": round(gb / (window_ms / 1e3), 1),
            "frac_of_hbm_peak": round(gb / (window_ms / 1e3) / HBM_PEAK_GBS, 4)}
    stages["scan_plus_posterior"] = scan_stage(need, mean)
    scan_gbs = stages["scan_plus_posterior"]["GBps"]
    dominant = max((k for k in ("scan", "bwd", "fwd_post", "beam", "sequence") if k in stages), key=lambda k: stages[k]["ms"])
    roofline = {"bound": "hbm", "kernel": dominant, "achieved": stages[dominant]["GBps"], "peak": HBM_PEAK_GBS,
                "unit": "GB/s", "frac": round(stages[dominant]["GBps"] / HBM_PEAK_GBS, 4),
                "traffic": measured_traffic(a.workload, N, a.columns, dominant)}

    # side measurements on the same batch (never `value`): the other arrangement of the scans, and the
    # hardware-exp/log scan arithmetic (not parity-grade)
    def side(split, mode, note):
        gpubuf.set_split_scans(split)
        gpubuf.set_scan_mode(mode)
        api.openfish_decode_gpu_discard(*call, gpubuf)
        ms, mn = timed_decodes(api, gpubuf, call, a.alt_steps)
        gpubuf.set_split_scans(asked)
        gpubuf.set_scan_mode(a.scan_mode)
        return {"chunks_per_s": round(N / (ms / 1e3), 1), "ms_per_step": round(ms, 4),
                "stage_ms": {k: round(v, 4) for k, v in mn.items() if v > 0},
                "scan_plus_posterior": scan_stage(need, mn), "note": note}

    other_split, fast_mode = None, None
    if a.alt_steps > 0:
        ran_split = mean["scan"] == 0  # what the timed calls ran with, asked for or chosen by the library
        other_split = side(not ran_split, a.scan_mode,
                           "split scans: backward scan, then forward scan + posterior on a second stream beside the beam search"
                           if not ran_split else "both scans and the posterior as one kernel, then the beam search")
        if a.scan_mode != "fast":
            fast_mode = side(asked, "fast",
                             "scans with v_exp_f32/v_log_f32 only: bwd within 2 ulp, a few posteriors per ten million "
                             "beyond 1e-3 relative; outside the acceptance bar, shown as the memory-bound floor of the kernels")

    # the same scores as the network emits them, five columns per state with a blank first (the layout
    # BASELINE's configurations name), read in place; its algorithmic bytes count C = 5 * 4^state_len
    five_columns = None
    if five is not None:
        scores5 = api.upload_scores_to_hip(five)
        del five
        call5 = (T, N, 5 * S, scores5, state_len, opt)
        api.openfish_decode_gpu_discard(*call5, gpubuf)
        ms5, mn5 = timed_decodes(api, gpubuf, call5, a.alt_steps)
        five_columns = {"C": 5 * S, "chunks_per_s": round(N / (ms5 / 1e3), 1), "ms_per_step": round(ms5, 4),
                        "stage_ms": {k: round(v, 4) for k, v in mn5.items() if v > 0},
                        "scan_plus_posterior": scan_stage(algorithmic_bytes(state_len, T, N, 5), mn5),
                        "note": "the same batch with five fp16 columns per state (blank first, never read), default settings"}
        scores5.free()

    # two batches in flight from one thread: enqueue on one gpubuf while the other one's decode
    # runs (the blocking call is enqueue + wait + copies into fresh host buffers)
    overlap = None
    if a.overlap_steps > 0:
        bufs = [gpubuf, api.GpuBuf(T, N, state_len)]
        bufs[1].set_scan_mode(a.scan_mode)
        bufs[1].set_split_scans(asked)
        api.openfish_decode_gpu(*call, bufs[1])
        t2 = time.perf_counter()
        api.openfish_amd_decode_enqueue(*call, bufs[0])
        for k in range(1, 2 * a.overlap_steps):
            api.openfish_amd_decode_enqueue(*call, bufs[k % 2])
            api.openfish_amd_decode_wait(bufs[(k - 1) % 2], copy=False)
        api.openfish_amd_decode_wait(bufs[(2 * a.overlap_steps - 1) % 2], copy=False)
        sec = time.perf_counter() - t2
        overlap = {"chunks_per_s": round(2 * a.overlap_steps * N / sec, 1), "gpubufs": 2,
                   "calls": 2 * a.overlap_steps,
                   "note": "one thread, openfish_amd_decode_enqueue/_wait alternating over two gpubufs, results "
                           "left in the pinned buffers; not `value`"}

    # what a plain streaming copy kernel reaches on this device (1 GiB each way, read + write
    # counted), as a second yardstick beside the published 8 TB/s.  Measured after the timed loops:
    # allocating and freeing the two large buffers first was seen to add 0.2 ms of host time to
    # every later decode call
    copy_gbs = None
    if a.copy_mib > 0:
        nbytes = a.copy_mib << 20
        src, dst = api.DeviceBuffer(nbytes), api.DeviceBuffer(nbytes)
        src.fill(1)
        api.lib().openfish_amd_copy(dst.ptr, src.ptr, nbytes)
        tc = time.perf_counter()
        for _ in range(5):
            api.lib().openfish_amd_copy(dst.ptr, src.ptr, nbytes)
        copy_gbs = 5 * 2 * nbytes / 1e9 / (time.perf_counter() - tc)
        src.free()
        dst.free()
    if copy_gbs:
        stages["device_copy_GBps"] = round(copy_gbs, 1)
        stages["scan_plus_posterior"]["frac_of_device_copy"] = round(scan_gbs / copy_gbs, 4)

    opt_kw = dict(beam_cut=100.0, blank_score=2.0, q_shift=q_shift, q_scale=q_scale)
    cpu = cpu_baseline(s16, state_len, opt_kw, min(a.cpu_sample, N)) if a.cpu_sample > 0 else None
    cpu1 = cpu_baseline_config1(a.seed) if a.cpu_sample > 0 else None

    print(json.dumps({
        "metric": "CRF chunks decoded/sec at %s (%d states, T=%d, N=%d); achieved HBM GB/s" % (a.workload, S, T, N),
        "value": round(N / (ms_per_step / 1e3), 1), "unit": "chunks/s", "n_gpus": 1, "steps": a.steps,
        "warmup": a.warmup, "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak",
        # state values and scores are fp32 (fp16 inputs); the default scans evaluate exp/log in fp64 where the
        # fp32 estimate is not provably the CPU path's result
        "vs_baseline": None, "dtype": "f32" if a.scan_mode == "fast" else "f32+f64", "data": "synthetic",
        "config": {"workload": "%s: state_len %d, S=%d, C=%d fp16 TNC (%d columns per state), T=%d, N=%d, beam 32, "
                               "beam_cut 100, blank 2.0" % (a.workload, state_len, S, C, a.columns, T, N),
                   "scan_mode": a.scan_mode, "scans": "one kernel" if mean["scan"] > 0 else "two kernels (backward, then forward + posterior beside the beam search)",
                   "seed": a.seed},
        "roofline": roofline, "stages": stages, "other_scan_arrangement": other_split, "fast_scan_mode": fast_mode,
        "five_columns": five_columns, "two_in_flight": overlap, "cpu_baseline": cpu, "cpu_baseline_config1": cpu1,
    }))


if __name__ == "__main__":
    main()
