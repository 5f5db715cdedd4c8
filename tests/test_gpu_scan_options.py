"""The scans under the settings no other GPU test exercises: stay scores other than 2.0, and
every states-per-lane choice in both scan arrangements and both parity-grade arithmetic modes.

Stay score.  openfish_decode_gpu hands options->blank_score to both scans, as the reference's GPU
path does (src/decode_hip.hip:120); the reference's CPU path adds the literal 2.0 whatever the
option says (src/decode_cpu.c:14,56), so no reference vector covers another value.  What pins the
GPU scans there: the closed form bwd[t] = (T - t) log(e^stay + 4 e^c) on constant scores, and the
oracle's scans with its stay knob set (pinned for that setting by the closed form and by dense
transition-matrix products, tests/test_oracle.py): bwd must be bit-identical, every posterior
within 1e-3 relative.
"""
import numpy as np
import pytest

from openfish_amd import synth
from oracle import crf_oracle as O

pytestmark = pytest.mark.gpu

RTOL = 1e-3
POST_ATOL = 1.2e-38


@pytest.fixture(scope="module")
def api():
    from openfish_amd import api as _api
    if _api.device_count() < 1:
        pytest.skip("no HIP device")
    return _api


def close(a, b):
    a, b = a.astype(np.float64), b.astype(np.float64)
    bad = np.abs(a - b) > RTOL * np.abs(b) + POST_ATOL
    assert not bad.any(), "%d of %d elements beyond 1e-3 relative" % (bad.sum(), bad.size)


def stage_scans(api, s16, state_len, stay, mode, fused):
    T, N, C = s16.shape
    S = 4 ** state_len
    sc = api.upload_scores_to_hip(s16)
    bwd = api.DeviceBuffer(4 * N * (T + 1) * S)
    post = api.DeviceBuffer(4 * N * (T + 1) * S)
    bwd.fill(0xFF)
    post.fill(0xFF)
    if fused:
        api.openfish_amd_scan_posterior(T, N, C, sc, state_len, stay, bwd, post, scan_mode=mode)
    else:
        api.openfish_amd_bwd_scan(T, N, C, sc, state_len, stay, bwd, scan_mode=mode)
        api.openfish_amd_fwd_post_scan(T, N, C, sc, state_len, stay, bwd, post, scan_mode=mode)
    return bwd.to_host(np.float32, (N, T + 1, S)), post.to_host(np.float32, (N, T + 1, S))


@pytest.mark.parametrize("stay", [0.5, -1.5, 5.0])
@pytest.mark.parametrize("state_len,T,N", [(3, 300, 5), (4, 200, 3), (5, 60, 2)])
def test_scans_with_other_stay_scores(api, stay, state_len, T, N):
    S = 4 ** state_len
    s16 = synth.crf_scores(T, N, state_len, seed=int(1000 + 10 * stay) + T)
    O.set_scan_stay(stay)
    try:
        ref_bwd, _, ref_post = O.scans(s16.astype(np.float32), state_len)
        kw = dict(blank_score=stay, q_scale=0.95, q_shift=-0.2)
        ref = O.decode(s16.astype(np.float32), state_len, kw, nthreads=4)
    finally:
        O.set_scan_stay()
    assert np.array_equal(ref["bwd"], ref_bwd)
    got = {}
    for fused in (False, True):
        for mode in ("two_tier", "precise"):
            bwd, post = stage_scans(api, s16, state_len, stay, api.SCAN_MODES[mode], fused)
            assert np.array_equal(bwd, ref_bwd), (fused, mode)
            close(post, ref_post)
            np.testing.assert_allclose(post.sum(axis=2), 1.0, rtol=2e-5)
            got[fused, mode] = post
    assert np.array_equal(got[False, "two_tier"], got[False, "precise"])
    assert np.array_equal(got[True, "two_tier"], got[True, "precise"])

    # the whole decode takes the option into its scans and into its beam search
    sc = api.upload_scores_to_hip(s16)
    gb = api.GpuBuf(T, N, state_len)
    for split in (False, True):
        gb.set_split_scans(split)
        mv, sq, qs = api.openfish_decode_gpu(T, N, 4 * S, sc, state_len, api.DECODER_INIT(**kw), gb)
        assert np.array_equal(gb.tensor("bwd_NTC"), ref_bwd)
        post = gb.tensor("post_NTC")
        close(post, ref_post)
        np.testing.assert_allclose(post.sum(axis=2), 1.0, rtol=2e-5)
        assert np.array_equal(mv, ref["moves"]) and np.array_equal(sq, ref["sequence"])


@pytest.mark.parametrize("stay", [0.5, -1.5, 5.0])
def test_constant_scores_closed_form_at_other_stay_scores(api, stay):
    T, N, sl, c = 96, 3, 4, -0.5
    S = 4 ** sl
    s16 = np.full((T, N, 4 * S), c, np.float16)
    per_step = np.log(np.exp(stay) + 4 * np.exp(c))
    want = (T - np.arange(T + 1)) * per_step
    for fused in (False, True):
        bwd, post = stage_scans(api, s16, sl, stay, api.SCAN_TWO_TIER, fused)
        np.testing.assert_allclose(bwd, np.broadcast_to(want[None, :, None], bwd.shape), rtol=2e-6, atol=1e-6)
        np.testing.assert_allclose(post, 1.0 / S, rtol=1e-5)


@pytest.mark.parametrize("split", [False, True])
@pytest.mark.parametrize("spl", [1, 2, 4])
@pytest.mark.parametrize("state_len,T,N", [(3, 257, 13), (4, 190, 7), (5, 70, 3)])
def test_every_states_per_lane_choice_gives_the_oracle_s_tensors(api, state_len, T, N, spl, split):
    """states per lane forced through the gpubuf's setter (the automatic choice depends on the batch
    size and never reaches most of them at test sizes), on small uneven batches, in both scan
    arrangements: bwd bit-identical to the oracle, the posterior within 1e-3, and the default
    arithmetic bit-identical to the always-double one (which is built with the fewest states per
    lane only and ignores the setter: the posteriors, whose normalising sum is taken in an order
    that depends on the lanes, are compared bit for bit where both ran with the same number)"""
    S = 4 ** state_len
    s16 = synth.crf_scores(T, N, state_len, seed=31 * spl + T, chunk_scale=synth.stress_scale(N) if state_len == 4 else None)
    ref_bwd, _, ref_post = O.scans(s16.astype(np.float32), state_len)
    sc = api.upload_scores_to_hip(s16)
    gb = api.GpuBuf(T, N, state_len)
    gb.set_scan_states_per_lane(spl)
    gb.set_split_scans(split)
    posts = {}
    for mode in ("two_tier", "precise"):
        gb.set_scan_mode(mode)
        api.openfish_decode_gpu(T, N, 4 * S, sc, state_len, api.DECODER_INIT(), gb)
        assert np.array_equal(gb.tensor("bwd_NTC"), ref_bwd), mode
        posts[mode] = gb.tensor("post_NTC")
        close(posts[mode], ref_post)
    fewest = 2 if state_len == 5 else 1
    used = max(spl, fewest) if (split or state_len != 3) else 1  # one kernel, 64 states: always one state per lane
    if used == fewest:
        assert np.array_equal(posts["two_tier"], posts["precise"])
