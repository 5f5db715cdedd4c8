"""Parity of the HIP path with the CPU oracle, through the C-ABI, on a real MI355X.

Tolerances (the acceptance bar of this decoder):
  * bwd and post tensors: |gpu - cpu| <= 1e-3 * |cpu| element-wise (for posteriors
    below the smallest normal fp32 number an absolute 1.2e-38 applies instead);
  * moves, sequence, qstring: identical bytes when the beam/sequence stage is fed
    the CPU path's own bwd/post tensors.
"""
import glob
import os

import numpy as np
import pytest

from openfish_amd import synth
from oracle import crf_oracle as O

pytestmark = pytest.mark.gpu

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")
CASES = sorted(os.path.basename(p)[:-4] for p in glob.glob(os.path.join(GOLDEN, "*.npz")))
GPU_CASES = [c for c in CASES if not c.startswith(("sl1", "sl2"))]  # the kernels cover 64, 256, 1024 states
RTOL = 1e-3
POST_ATOL = 1.2e-38


@pytest.fixture(scope="module")
def api():
    from openfish_amd import api as _api
    if _api.device_count() < 1:
        pytest.skip("no HIP device")
    return _api


def load(name):
    z = np.load(os.path.join(GOLDEN, name + ".npz"))
    bc, bl, qs, qc = [float(v) for v in z["opt"]]
    return z, int(z["state_len"]), dict(beam_cut=bc, blank_score=bl, q_shift=qs, q_scale=qc)


def close(a, b, atol=0.0):
    a, b = a.astype(np.float64), b.astype(np.float64)
    bad = np.abs(a - b) > RTOL * np.abs(b) + atol
    assert not bad.any(), "%d of %d elements beyond 1e-3 relative, worst %.3e" % (
        bad.sum(), bad.size, (np.abs(a - b) / np.maximum(np.abs(b), 1e-300)).max())


def qstring_close(qs, want, moves):
    """Whole-decode bound on the phred string.  moves and sequence of a whole decode equal the CPU
    path's; a quality character comes from a posterior that agrees with the CPU path's to about
    2e-6 relative (the CPU path sums the 4^state_len exponentials of a time step one by one in
    fp32, the GPU by a tree), which moves a base's quality across a character boundary now and
    then: at most one phred step, on at most 0.5 % of the bases (about 0.05 % is typical)."""
    diff = qs.astype(np.int16) - want.astype(np.int16)
    assert np.abs(diff).max() <= 1, "a phred character is off by %d steps" % np.abs(diff).max()
    bases = int(moves.sum())
    assert np.count_nonzero(diff) <= max(1, bases // 200), "%d of %d phred characters differ" % (
        np.count_nonzero(diff), bases)


def gpu_scans(api, s16, state_len, stay=2.0, mode="two_tier"):
    T, N, C = s16.shape
    S = 4 ** state_len
    sc = api.upload_scores_to_hip(s16)
    bwd = api.DeviceBuffer(4 * N * (T + 1) * S)
    post = api.DeviceBuffer(4 * N * (T + 1) * S)
    bwd.fill(0xFF)
    post.fill(0xFF)
    api.openfish_amd_bwd_scan(T, N, C, sc, state_len, stay, bwd, scan_mode=mode)
    api.openfish_amd_fwd_post_scan(T, N, C, sc, state_len, stay, bwd, post, scan_mode=mode)
    return bwd.to_host(np.float32, (N, T + 1, S)), post.to_host(np.float32, (N, T + 1, S))


def gpu_scan_posterior(api, s16, state_len, stay=2.0, mode="two_tier"):
    """both scans and the posterior as one kernel"""
    T, N, C = s16.shape
    S = 4 ** state_len
    sc = api.upload_scores_to_hip(s16)
    bwd = api.DeviceBuffer(4 * N * (T + 1) * S)
    post = api.DeviceBuffer(4 * N * (T + 1) * S)
    bwd.fill(0xFF)
    post.fill(0xFF)
    api.openfish_amd_scan_posterior(T, N, C, sc, state_len, stay, bwd, post, scan_mode=mode)
    return bwd.to_host(np.float32, (N, T + 1, S)), post.to_host(np.float32, (N, T + 1, S))


def gpu_from_tensors(api, s16, state_len, opt_kw, bwd, post, debug_flags=0):
    T, N, C = s16.shape
    sc = api.upload_scores_to_hip(s16)
    gb = api.GpuBuf(T, N, state_len)
    gb.set_debug_flags(debug_flags)
    rb, rp = api.DeviceBuffer.from_host(bwd), api.DeviceBuffer.from_host(post)
    out = api.openfish_amd_decode_from_tensors(T, N, C, sc, state_len, api.DECODER_INIT(**opt_kw), rb, rp, gb)
    return out, gb


# ---- golden vectors written by the compiled reference ---------------------------

@pytest.mark.parametrize("name", GPU_CASES)
def test_scans_match_reference_golden(api, name):
    z, sl, opt = load(name)
    for scans in (gpu_scans, gpu_scan_posterior):
        bwd, post = scans(api, z["scores"], sl)
        close(bwd, z["bwd"])
        close(post, z["post"], POST_ATOL)
        assert np.array_equal(bwd, z["bwd"])  # stronger than the bar: the CPU path's roundings are reproduced


@pytest.mark.parametrize("name", GPU_CASES)
def test_beam_stage_bit_exact_on_reference_tensors(api, name):
    z, sl, opt = load(name)
    (mv, sq, qs), gb = gpu_from_tensors(api, z["scores"], sl, opt, z["bwd"], z["post"])
    assert np.array_equal(mv, z["moves"])
    assert np.array_equal(sq, z["sequence"])
    assert np.array_equal(qs, z["qstring"])
    assert np.array_equal(gb.tensor("total_probs"), z["total_probs"]) or \
        np.allclose(gb.tensor("total_probs"), z["total_probs"], rtol=3e-7)
    np.testing.assert_allclose(gb.tensor("qual_data"), z["qual_data"], rtol=3e-7)  # pow: last bit of libm


@pytest.mark.parametrize("name", GPU_CASES)
def test_quality_from_per_state_sums_equals_quality_from_gathers(api, name):
    """the quality stage reads the posteriors behind a block either by itself (nine gathers per time
    step: the stage-level entry point, and a decode with split scans) or as one value per time step
    from the per-state sums a kernel leaves beside the beam search (a whole decode of up to 512
    chunks of 64 or 256 states, and the decode from given tensors): the same fp32 sums in the same
    order, so every output of the stage is identical bit for bit"""
    z, sl, opt = load(name)
    T, N, C = z["scores"].shape
    (mv, sq, qs), gb = gpu_from_tensors(api, z["scores"], sl, opt, z["bwd"], z["post"])
    with_sums = {k: gb.tensor(k) for k in ("qual_data", "base_probs", "total_probs", "sequence", "qstring")}
    gb2 = api.GpuBuf(T, N, sl)
    sc = api.upload_scores_to_hip(z["scores"])
    rb, rp = api.DeviceBuffer.from_host(z["bwd"]), api.DeviceBuffer.from_host(z["post"])
    o = api.DECODER_INIT(**opt)
    api.openfish_amd_beam_search(T, N, C, sc, sl, o, rb, gb2)
    api.openfish_amd_sequence(T, N, sl, o, rp, gb2)
    for k, v in with_sums.items():
        assert np.array_equal(v.view(np.uint8), gb2.tensor(k).view(np.uint8)), k
    assert np.array_equal(sq, gb2.tensor("sequence")) and np.array_equal(qs, gb2.tensor("qstring"))


@pytest.mark.parametrize("name", GPU_CASES)
def test_whole_decode_on_golden(api, name):
    """openfish_decode_gpu end to end; with the CPU-faithful scan arithmetic the GPU's own
    tensors lead to the same calls as the reference's"""
    z, sl, opt = load(name)
    s16 = z["scores"]
    T, N, C = s16.shape
    if opt["blank_score"] != 2.0:
        pytest.skip("the CPU scans ignore blank_score, the GPU entry point does not (as in the reference)")
    sc = api.upload_scores_to_hip(s16)
    gb = api.GpuBuf(T, N, sl)
    for split in (None, False, True):  # the library's choice for the batch, one kernel, two kernels
        gb.set_split_scans(split)
        mv, sq, qs = api.openfish_decode_gpu(T, N, C, sc, sl, api.DECODER_INIT(**opt), gb)
        assert np.array_equal(mv, z["moves"]) and np.array_equal(sq, z["sequence"]) and np.array_equal(qs, z["qstring"])
        t = gb.timings()
        assert set(t) == set(api.STAGES) and t["beam"] > 0 and t["sequence"] > 0 and t["total"] > 0
        ran_split = t["scan"] == 0
        if ran_split:  # the sums follow the forward kernel where they fit beside the search: 64 states
            assert t["bwd"] > 0 and t["fwd_post"] > 0 and (t["path_sums"] > 0) == (sl == 3 and N <= 512)
        else:
            assert t["bwd"] == 0 and t["fwd_post"] == 0 and (t["path_sums"] > 0) == (sl <= 4 and N <= 512)
        if split is None:  # small batches of up to 256 states run split
            assert ran_split == (sl <= 4 and N * 4 ** sl <= 512 * 256)
        else:
            assert ran_split == split


def test_reference_in_repo_fixture_end_to_end(api):
    """the reference's own known-answer test (fast model, N=1, T=1666); its fp32 scores are
    all exactly representable in fp16"""
    sc32 = np.fromfile(os.path.join(GOLDEN, "ref_fixture_scores.blob"), np.float32).reshape(1666, 1, 256)
    s16 = sc32.astype(np.float16)
    assert np.array_equal(s16.astype(np.float32), sc32)
    sc = api.upload_scores_to_hip(s16)
    gb = api.GpuBuf(1666, 1, 3)
    mv, sq, qs = api.openfish_decode_gpu(1666, 1, 256, sc, 3, api.DECODER_INIT(q_scale=0.97, q_shift=-1.8), gb)
    for got, name in ((mv, "moves"), (sq, "sequence"), (qs, "qstring")):
        want = np.fromfile(os.path.join(GOLDEN, "ref_fixture_%s.blob" % name), np.uint8).reshape(1, 1666)
        assert np.array_equal(got, want), name


# ---- seeded inputs against the oracle ----------------------------------------------

SHAPES = [
    # state_len, T, N, stress
    (3, 1, 1, False), (3, 2, 3, False), (3, 7, 5, False), (3, 9, 4, True), (3, 333, 13, True),
    (4, 1, 2, False), (4, 5, 1, False), (4, 257, 9, False), (4, 130, 6, True),
    (5, 3, 1, False), (5, 61, 3, False), (5, 40, 2, True),
    # more than 512 chunks: the beam search runs four chunks to a workgroup, the last group ragged
    (3, 24, 517, False), (4, 12, 514, True),
    # long chunks: the sequence stage's per-chunk tables beyond 64 KB of LDS, and the longest allowed
    (3, 4700, 2, False), (4, 8192, 1, False),
]


@pytest.mark.parametrize("state_len,T,N,stress", SHAPES)
def test_stages_against_oracle(api, state_len, T, N, stress):
    """ragged shapes: T below the prefetch depth, N not a multiple of the chunks a
    workgroup holds, single chunks"""
    scale = synth.stress_scale(N) if stress else None
    s16 = synth.crf_scores(T, N, state_len, seed=1000 + 7 * T + N, chunk_scale=scale)
    kw = dict(q_scale=0.95, q_shift=-0.2)
    ref = O.decode(s16.astype(np.float32), state_len, kw, nthreads=4)
    for scans in (gpu_scans, gpu_scan_posterior):
        bwd, post = scans(api, s16, state_len)
        assert np.array_equal(bwd, ref["bwd"])
        close(post, ref["post"], POST_ATOL)
        assert np.all(bwd[:, T, :] == 0.0)
    (mv, sq, qs), gb = gpu_from_tensors(api, s16, state_len, kw, ref["bwd"], ref["post"])
    assert np.array_equal(mv, ref["moves"])
    assert np.array_equal(gb.tensor("states"), ref["states"])
    assert np.array_equal(sq, ref["sequence"])
    assert np.array_equal(qs, ref["qstring"])


@pytest.mark.parametrize("seed", [101, 102, 103])
def test_random_shapes_and_options_beam_stage_bit_exact(api, seed):
    """random model size, shape, per-chunk score scale (flat to peaked), beam cut (none to very
    tight), stay score and quality options: the stages after the scans, fed the CPU path's
    tensors, reproduce the CPU path's bytes"""
    rng = np.random.default_rng(seed)
    for _ in range(25):
        sl = int(rng.choice([3, 3, 4, 4, 5]))
        T = int(rng.integers(1, 260)) if sl < 5 else int(rng.integers(1, 90))
        N = int(rng.integers(1, 9))
        scale = rng.choice([0.05, 0.3, 1.0, 2.5, 8.0], size=N).astype(np.float32)
        s16 = synth.crf_scores(T, N, sl, seed=int(rng.integers(1 << 30)), chunk_scale=scale)
        kw = dict(beam_cut=float(rng.choice([0.0, 0.5, 3.0, 17.0, 100.0, 1e6])),
                  blank_score=float(rng.choice([2.0, 0.0, -1.5, 5.0])),
                  q_scale=float(rng.choice([1.0, 0.95, 1.3])), q_shift=float(rng.choice([0.0, -0.2, 4.0])))
        ref = O.decode(s16.astype(np.float32), sl, kw, nthreads=4)
        (mv, sq, qs), _ = gpu_from_tensors(api, s16, sl, kw, ref["bwd"], ref["post"])
        what = (sl, T, N, scale.tolist(), kw)
        assert np.array_equal(mv, ref["moves"]), what
        assert np.array_equal(sq, ref["sequence"]), what
        assert np.array_equal(qs, ref["qstring"]), what


@pytest.mark.parametrize("seed", [201, 202])
def test_random_shapes_whole_decode(api, seed):
    """the same kind of random cases through openfish_decode_gpu (four- and five-column input, both
    scans as one kernel or split): bwd identical, posterior within tolerance, moves and sequence
    identical, phred string within the bound of qstring_close"""
    rng = np.random.default_rng(seed)
    for _ in range(20):
        sl = int(rng.choice([3, 4, 4, 5]))
        T = int(rng.integers(1, 400)) if sl < 5 else int(rng.integers(1, 120))
        N = int(rng.integers(1, 11))
        S = 4 ** sl
        scale = rng.choice([0.05, 0.3, 1.0, 2.5, 6.0], size=N).astype(np.float32)
        five = bool(rng.integers(2))
        out = synth.crf_scores(T, N, sl, seed=int(rng.integers(1 << 30)), chunk_scale=scale, five_columns=five)
        four, dev_in = (out[0], out[1]) if five else (out, out)
        kw = dict(beam_cut=float(rng.choice([3.0, 100.0, 1e6])), q_scale=0.95, q_shift=-0.2)
        ref = O.decode(four.astype(np.float32), sl, kw, nthreads=4)
        gb = api.GpuBuf(T, N, sl)
        sc = api.upload_scores_to_hip(dev_in)
        gb.set_split_scans(bool(rng.integers(2)))
        mv, sq, qs = api.openfish_decode_gpu(T, N, (5 if five else 4) * S, sc, sl, api.DECODER_INIT(**kw), gb)
        what = (sl, T, N, five, scale.tolist(), kw)
        assert np.array_equal(gb.tensor("bwd_NTC"), ref["bwd"]), what
        close(gb.tensor("post_NTC"), ref["post"], POST_ATOL)
        assert np.array_equal(mv, ref["moves"]), what
        assert np.array_equal(sq, ref["sequence"]), what
        qstring_close(qs, ref["qstring"], mv)


@pytest.mark.parametrize("state_len,T,N,five", [(4, 96, 2048, False), (4, 40, 2048, True), (3, 50, 2100, False),
                                                 (5, 24, 512, False)])
def test_batches_whose_rows_lie_4_mib_apart_whole_decode(api, state_len, T, N, five):
    """short chunks in batches where one time step of the scores is 4 MiB (2048 chunks of 256 states, 512 of
    1024; 5 MiB with five columns), the spacing at which the rows a workgroup keeps in flight share DRAM
    banks, and beyond 2048 chunks of 64 states: in every arrangement setting the whole decode gives the
    oracle's bwd, moves and sequence, posteriors within tolerance, phred string within qstring_close"""
    S = 4 ** state_len
    out = synth.crf_scores(T, N, state_len, seed=77 + N + T, chunk_scale=synth.stress_scale(N), five_columns=five,
                           threads=16)
    four, dev_in = (out[0], out[1]) if five else (out, out)
    kw = dict(q_scale=0.95, q_shift=-0.2)
    ref = O.decode(four.astype(np.float32), state_len, kw, nthreads=16)
    gb = api.GpuBuf(T, N, state_len)
    sc = api.upload_scores_to_hip(dev_in)
    for split in (None, False, True):
        gb.set_split_scans(split)
        mv, sq, qs = api.openfish_decode_gpu(T, N, (5 if five else 4) * S, sc, state_len, api.DECODER_INIT(**kw), gb)
        assert np.array_equal(gb.tensor("bwd_NTC"), ref["bwd"]), split
        close(gb.tensor("post_NTC"), ref["post"], POST_ATOL)
        assert np.array_equal(mv, ref["moves"]) and np.array_equal(sq, ref["sequence"]), split
        qstring_close(qs, ref["qstring"], mv)


def test_fast_scan_mode_stays_within_two_ulp_of_bwd(api):
    """the hardware-exp/log scans are a measurement aid, not a parity-grade mode: bwd within 2 ulp
    of the CPU path, and a posterior may leave the 1e-3 bar (only a loose bound is asserted)"""
    s16 = synth.crf_scores(400, 6, 4, seed=77)
    ref = O.scans(s16.astype(np.float32), 4)
    bwd, post = gpu_scans(api, s16, 4, mode="fast")
    np.testing.assert_allclose(bwd, ref[0], rtol=3e-7)
    np.testing.assert_allclose(post, ref[2], rtol=5e-3, atol=POST_ATOL)


@pytest.mark.parametrize("state_len,T,N,stress", [(3, 700, 9, False), (4, 900, 6, True), (5, 300, 2, False)])
def test_two_tier_and_precise_scans_are_bit_identical(api, state_len, T, N, stress):
    """the default two-tier arithmetic and the always-double arithmetic must give the same bits
    (both are the CPU path's bwd; the posterior only differs through bwd and fwd)"""
    scale = synth.stress_scale(N) if stress else None
    s16 = synth.crf_scores(T, N, state_len, seed=88 + T, chunk_scale=scale)
    b2, p2 = gpu_scans(api, s16, state_len, mode="two_tier")
    b1, p1 = gpu_scans(api, s16, state_len, mode="precise")
    assert np.array_equal(b2, b1)
    assert np.array_equal(p2, p1)
    b3, p3 = gpu_scan_posterior(api, s16, state_len, mode="two_tier")
    b4, p4 = gpu_scan_posterior(api, s16, state_len, mode="precise")
    assert np.array_equal(b3, b1) and np.array_equal(b4, b1)
    assert np.array_equal(p3, p4)
    np.testing.assert_allclose(p3, p1, rtol=1e-5, atol=POST_ATOL)  # another exponent shift, another sum order


def test_serial_merge_route_gives_identical_output(api):
    """the route taken after a CRC collision (serial replay of the merges) must agree with
    the parallel one whenever there is no collision"""
    s16 = synth.crf_scores(300, 9, 4, seed=31, chunk_scale=synth.stress_scale(9))
    kw = dict(q_scale=0.95, q_shift=-0.2)
    ref = O.decode(s16.astype(np.float32), 4, kw, nthreads=4)
    (mv, sq, qs), _ = gpu_from_tensors(api, s16, 4, kw, ref["bwd"], ref["post"], debug_flags=1)
    assert np.array_equal(mv, ref["moves"]) and np.array_equal(sq, ref["sequence"]) and np.array_equal(qs, ref["qstring"])


def test_options_beam_cut_and_blank_score(api):
    s16 = synth.crf_scores(250, 5, 3, seed=41)
    for kw in (dict(beam_cut=3.0), dict(beam_cut=1e6, blank_score=0.5), dict(beam_cut=0.0), dict(q_scale=1.3, q_shift=4.0)):
        ref = O.decode(s16.astype(np.float32), 3, kw, nthreads=4)
        (mv, sq, qs), _ = gpu_from_tensors(api, s16, 3, kw, ref["bwd"], ref["post"])
        assert np.array_equal(mv, ref["moves"]), kw
        assert np.array_equal(sq, ref["sequence"]), kw
        assert np.array_equal(qs, ref["qstring"]), kw


def test_gpubuf_is_reusable_for_smaller_batches(api):
    gb = api.GpuBuf(200, 8, 3)
    for T, N, seed in ((200, 8, 1), (77, 3, 2), (200, 8, 1)):
        s16 = synth.crf_scores(T, N, 3, seed=seed)
        ref = O.decode(s16.astype(np.float32), 3, nthreads=4)
        sc = api.upload_scores_to_hip(s16)
        mv, sq, qs = api.openfish_decode_gpu(T, N, 4 * 64, sc, 3, api.DECODER_INIT(), gb)
        assert np.array_equal(mv, ref["moves"]) and np.array_equal(sq, ref["sequence"]) and np.array_equal(qs, ref["qstring"])


def test_enqueue_and_wait_with_two_batches_in_flight(api):
    """two gpubufs, both decodes queued before either is waited for, twice over; results as
    the oracle's (and so as the blocking call's)"""
    kw = dict(q_scale=0.95, q_shift=-0.2)
    opt = api.DECODER_INIT(**kw)
    shapes = ((4, 300, 7), (3, 420, 9))
    bufs = [api.GpuBuf(T, N, sl) for sl, T, N in shapes]
    for rnd in range(2):
        inputs = [synth.crf_scores(T, N, sl, seed=600 + 10 * rnd + k) for k, (sl, T, N) in enumerate(shapes)]
        dev = [api.upload_scores_to_hip(x) for x in inputs]
        for (sl, T, N), sc, gb in zip(shapes, dev, bufs):
            api.openfish_amd_decode_enqueue(T, N, 4 * 4 ** sl, sc, sl, opt, gb)
        for (sl, T, N), x, gb in zip(shapes, inputs, bufs):
            mv, sq, qs = api.openfish_amd_decode_wait(gb)
            ref = O.decode(x.astype(np.float32), sl, kw, nthreads=4)
            assert np.array_equal(mv, ref["moves"]) and np.array_equal(sq, ref["sequence"])
            assert np.array_equal(qs, ref["qstring"])
            assert set(gb.timings()) >= {"bwd", "beam"}
        del dev


@pytest.mark.parametrize("state_len,T,N", [(3, 150, 5), (4, 90, 3), (5, 40, 2), (4, 333, 40), (3, 64, 9), (3, 1, 2), (4, 2, 1),
                                           (5, 3, 1)])
def test_five_column_input_equals_its_four_column_view(api, state_len, T, N):
    """C = 5*S: a blank column in front of the four step columns of every state, read where it
    lies by every kernel that takes scores; the blank values (poisoned here) are never looked at"""
    S = 4 ** state_len
    four, five = synth.crf_scores(T, N, state_len, seed=55, five_columns=True)
    assert np.array_equal(five.reshape(T, N, S, 5)[..., 1:].reshape(T, N, 4 * S), four)
    five = five.copy()
    five.reshape(T, N, S, 5)[..., 0] = np.float16(np.nan)
    kw = dict(q_scale=0.95, q_shift=-0.2)
    ref = O.decode(four.astype(np.float32), state_len, kw, nthreads=4)
    gb = api.GpuBuf(T, N, state_len)
    sc5 = api.upload_scores_to_hip(five)
    for split in (False, True):
        gb.set_split_scans(split)
        mv, sq, qs = api.openfish_decode_gpu(T, N, 5 * S, sc5, state_len, api.DECODER_INIT(**kw), gb)
        assert np.array_equal(gb.tensor("bwd_NTC"), ref["bwd"])
        close(gb.tensor("post_NTC"), ref["post"], POST_ATOL)
        assert np.array_equal(mv, ref["moves"]) and np.array_equal(sq, ref["sequence"])
        assert np.array_equal(qs, ref["qstring"])
    # the stages one by one, every scan mode
    for mode in ("two_tier", "precise", "fast"):
        for scans in (gpu_scans, gpu_scan_posterior):
            bwd, post = scans(api, five, state_len, mode=mode)
            if mode == "fast":
                np.testing.assert_allclose(bwd, ref["bwd"], rtol=3e-7, atol=1e-6)
            else:
                assert np.array_equal(bwd, ref["bwd"])
                close(post, ref["post"], POST_ATOL)
    (mv, sq, qs), _ = gpu_from_tensors(api, five, state_len, kw, ref["bwd"], ref["post"])
    assert np.array_equal(mv, ref["moves"]) and np.array_equal(sq, ref["sequence"]) and np.array_equal(qs, ref["qstring"])
    (mv, sq, qs), _ = gpu_from_tensors(api, five, state_len, kw, ref["bwd"], ref["post"], debug_flags=1)
    assert np.array_equal(mv, ref["moves"]) and np.array_equal(sq, ref["sequence"]) and np.array_equal(qs, ref["qstring"])


@pytest.mark.parametrize("state_len,T,N", [(4, 240, 6), (3, 300, 8), (5, 90, 2)])
def test_duplicate_hashes_are_detected_and_merged_like_the_cpu_path(api, state_len, T, N):
    """Beam elements whose sequences differ but whose hashes are equal (a CRC collision): forced
    here by seeding the beam with hashes of (state & 15) on both sides.  A stay then finds several
    equal hashes, and one step is claimed by two stays; the search has to notice that on its own
    (no replay flag) and fall back to the CPU path's merge order."""
    s16 = synth.crf_scores(T, N, state_len, seed={240: 2, 300: 4542, 90: 4332}[T])
    kw = dict(q_scale=0.95, q_shift=-0.2)
    plain = O.decode(s16.astype(np.float32), state_len, kw, nthreads=4)
    O.set_seed_state_mask(15)
    try:
        ref = O.decode_from_tensors(s16.astype(np.float32), state_len, plain["bwd"], plain["post"], kw, nthreads=4)
    finally:
        O.set_seed_state_mask()
    assert not np.array_equal(ref["moves"], plain["moves"]), "the shared hashes changed nothing: the case is too tame"
    (mv, sq, qs), _ = gpu_from_tensors(api, s16, state_len, kw, plain["bwd"], plain["post"], debug_flags=2)
    assert np.array_equal(mv, ref["moves"]) and np.array_equal(sq, ref["sequence"]) and np.array_equal(qs, ref["qstring"])
    (mv, sq, qs), _ = gpu_from_tensors(api, s16, state_len, kw, plain["bwd"], plain["post"], debug_flags=3)
    assert np.array_equal(mv, ref["moves"]) and np.array_equal(sq, ref["sequence"]) and np.array_equal(qs, ref["qstring"])


def test_two_threads_with_a_gpubuf_each_keep_their_own_settings(api):
    """settings live in the gpubuf: a thread decoding with the hardware-exp scans and split kernels
    does not change what a thread with the default settings gets, and the other way round"""
    import threading
    sl, T, N = 4, 500, 12
    S = 4 ** sl
    s16 = synth.crf_scores(T, N, sl, seed=314, chunk_scale=synth.stress_scale(N))
    kw = dict(q_scale=0.95, q_shift=-0.2)
    sc = api.upload_scores_to_hip(s16)
    opt = api.DECODER_INIT(**kw)

    def decode_with(mode, split, flags):
        gb = api.GpuBuf(T, N, sl)
        gb.set_scan_mode(mode)
        gb.set_split_scans(split)
        gb.set_debug_flags(flags)
        out = api.openfish_decode_gpu(T, N, 4 * S, sc, sl, opt, gb)
        return out, gb.tensor("bwd_NTC")

    want = {"a": decode_with("two_tier", False, 0), "b": decode_with("fast", True, 1)}
    assert not np.array_equal(want["a"][1], want["b"][1]), "the two settings should differ in the last bits of bwd"
    got, errors = {"a": [], "b": []}, []

    def worker(key, mode, split, flags):
        try:
            api.lib().set_device_hip(0)
            for _ in range(6):
                got[key].append(decode_with(mode, split, flags))
        except Exception as e:  # surfaced below: an exception in a thread would otherwise pass silently
            errors.append(e)

    threads = [threading.Thread(target=worker, args=("a", "two_tier", False, 0)),
               threading.Thread(target=worker, args=("b", "fast", True, 1))]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    assert not errors, errors
    for key in ("a", "b"):
        assert len(got[key]) == 6
        for (mv, sq, qs), bwd in got[key]:
            assert np.array_equal(bwd, want[key][1])
            assert np.array_equal(mv, want[key][0][0]) and np.array_equal(sq, want[key][0][1])
            assert np.array_equal(qs, want[key][0][2])


def test_constant_scores_closed_form(api):
    T, N, sl, c = 64, 3, 3, 0.75
    S = 4 ** sl
    s16 = np.full((T, N, 4 * S), c, np.float16)
    bwd, post = gpu_scans(api, s16, sl)
    per_step = np.log(np.exp(2.0) + 4 * np.exp(c))
    want = (T - np.arange(T + 1)) * per_step
    np.testing.assert_allclose(bwd, np.broadcast_to(want[None, :, None], bwd.shape), rtol=2e-6)
    np.testing.assert_allclose(post, 1.0 / S, rtol=1e-5)


# ---- full benchmark sizes: every chunk against the oracle, plus size-independent properties ----

FULL = [("fast", 3, 1666, 512, False, 4), ("hac", 4, 1666, 512, False, 4),
        ("sup", 5, 1666, 256, False, 4), ("hac_stress", 4, 1666, 1024, True, 4),
        ("fast_five_columns", 3, 1666, 512, False, 5), ("hac_five_columns", 4, 1666, 512, False, 5),
        ("sup_five_columns", 5, 1666, 256, False, 5), ("hac_stress_five_columns", 4, 1666, 1024, True, 5)]


@pytest.mark.parametrize("name,state_len,T,N,stress,columns", FULL)
def test_full_size_configurations(api, name, state_len, T, N, stress, columns):
    """the benchmark configurations at full size (scores with four columns per state, and with
    the five the network emits), all N chunks: bwd bit-identical to the
    oracle, every posterior within 1e-3 relative, whole-decode moves and sequence identical and
    the phred string within its bound; then the beam/sequence stage fed the oracle's tensors,
    identical bytes for all N chunks"""
    S, C = 4 ** state_len, columns * 4 ** state_len
    scale = synth.stress_scale(N) if stress else None
    made = synth.crf_scores(T, N, state_len, seed=2025, chunk_scale=scale, threads=16, five_columns=columns == 5)
    s16, given = (made[0], made[1]) if columns == 5 else (made, made)  # s16: what the oracle decodes
    kw = dict(q_scale=0.95, q_shift=-0.2)
    sc = api.upload_scores_to_hip(given)
    gb = api.GpuBuf(T, N, state_len)
    mv, sq, qs = api.openfish_decode_gpu(T, N, C, sc, state_len, api.DECODER_INIT(**kw), gb)

    # size-independent properties of every chunk
    assert mv.shape == (N, T) and set(np.unique(mv)) <= {0, 1} and np.all(mv[:, 0] == 1)
    lens = mv.sum(axis=1)
    pos = np.arange(T)[None, :]
    inside = pos < lens[:, None]
    assert np.all(np.isin(sq[inside], np.frombuffer(b"ACGT", np.uint8))) and np.all(sq[~inside] == 0)
    assert np.all((qs[inside] >= 34) & (qs[inside] <= 83)) and np.all(qs[~inside] == 0)

    # the oracle on all N chunks, compared in slabs of chunks to bound host memory
    ref = O.decode(s16.astype(np.float32), state_len, kw, nthreads=16)
    bwd, post = gb.tensor("bwd_NTC"), gb.tensor("post_NTC")
    step = 64
    for lo in range(0, N, step):
        hi = min(N, lo + step)
        assert np.array_equal(bwd[lo:hi], ref["bwd"][lo:hi]), "bwd differs in chunks %d..%d" % (lo, hi)
        close(post[lo:hi], ref["post"][lo:hi], POST_ATOL)
        np.testing.assert_allclose(post[lo:hi].sum(axis=2), 1.0, rtol=2e-5)
    assert np.array_equal(mv, ref["moves"]) and np.array_equal(sq, ref["sequence"])
    qstring_close(qs, ref["qstring"], mv)
    del bwd, post

    # the split scans give the same bwd bits and the same posterior up to the last digits
    gb.set_split_scans(True)
    mv1, sq1, qs1 = api.openfish_decode_gpu(T, N, C, sc, state_len, api.DECODER_INIT(**kw), gb)
    assert np.array_equal(gb.tensor("bwd_NTC"), ref["bwd"])
    assert np.array_equal(mv1, mv) and np.array_equal(sq1, sq)
    qstring_close(qs1, ref["qstring"], mv)

    # beam search + sequence stage on the oracle's own tensors: identical bytes, every chunk
    (mv2, sq2, qs2), _ = gpu_from_tensors(api, given, state_len, kw, ref["bwd"], ref["post"])
    assert np.array_equal(mv2, ref["moves"]) and np.array_equal(sq2, ref["sequence"]) and np.array_equal(qs2, ref["qstring"])


# ---- rotary embedding ------------------------------------------------------------------

@pytest.mark.parametrize("batch,seqlen,nheads,head_dim,half", [(3, 17, 4, 16, 8), (2, 33, 8, 64, 32),
                                                                (2, 5, 3, 10, 3), (1, 1, 1, 2, 1),
                                                                (16, 833, 8, 64, 32)])
def test_rotary_matches_cpu_path_rounded_to_half(api, batch, seqlen, nheads, head_dim, half):
    rng = np.random.default_rng(batch * 100 + seqlen)
    x16 = rng.standard_normal((batch, seqlen, nheads, head_dim)).astype(np.float16)
    sn, cs = synth.rotary_tables(seqlen, half)
    strides = (seqlen * nheads * head_dim, nheads * head_dim, head_dim)
    want = O.rotary_emb(x16.astype(np.float32), sn, cs, batch, seqlen, nheads, head_dim, half, *strides)
    want16 = want.reshape(x16.shape).astype(np.float16)
    xd = api.DeviceBuffer.from_host(x16)
    sd, cd = api.DeviceBuffer.from_host(sn), api.DeviceBuffer.from_host(cs)
    api.openfish_rotary_emb_gpu(xd, sd, cd, batch, seqlen, nheads, head_dim, half, *strides)
    got = xd.to_host(np.float16, x16.shape)
    assert np.array_equal(got.view(np.uint16), want16.view(np.uint16))
    assert np.array_equal(got[..., 2 * half:], x16[..., 2 * half:])  # beyond the rotary span: untouched
