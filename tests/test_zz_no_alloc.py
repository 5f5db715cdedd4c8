"""The beam search entry point that allocates nothing (its scratch is a static device array of
the library) against the entry point that works on a gpubuf, through the C-ABI: same states and
moves, bit for bit, on two calls in a row, the second one smaller; and the amount of free device
memory is the same before and after a call."""
import numpy as np
import pytest

from openfish_amd import synth

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def api():
    from openfish_amd import api as _api
    if _api.device_count() < 1:
        pytest.skip("no HIP device")
    return _api


def both_entry_points(api, state_len, T, N, seed, scale=None, columns=4, **opt_kw):
    S = 4 ** state_len
    C = columns * S
    s16 = synth.crf_scores(T, N, state_len, seed=seed, chunk_scale=scale, five_columns=columns == 5)
    if columns == 5:
        s16 = s16[1]
    sc = api.upload_scores_to_hip(s16)
    bwd = api.DeviceBuffer(4 * N * (T + 1) * S)
    api.openfish_amd_bwd_scan(T, N, C, sc, state_len, 2.0, bwd)
    opt = api.DECODER_INIT(**opt_kw)

    gb = api.GpuBuf(T, N, state_len)
    api.openfish_amd_beam_search(T, N, C, sc, state_len, opt, bwd, gb)
    want_states, want_moves = gb.tensor("states"), gb.tensor("moves")

    states, moves = api.DeviceBuffer(4 * N * T), api.DeviceBuffer(N * T)
    states.fill(0xEE)
    moves.fill(0xEE)
    api.openfish_amd_beam_search_static_prepare()  # once per device; later calls return at once
    api.lib().openfish_amd_sync()
    free_before = api.device_free_bytes()
    api.openfish_amd_beam_search_static(T, N, C, sc, state_len, opt, bwd, states, moves)  # launches and returns
    api.lib().openfish_amd_sync()
    assert api.device_free_bytes() == free_before, "the call changed the amount of free device memory"
    got_states, got_moves = states.to_host(np.int32, (N, T)), moves.to_host(np.uint8, (N, T))
    assert np.array_equal(got_moves, want_moves)
    assert np.array_equal(got_states, want_states)
    assert got_moves[:, 0].all() and set(np.unique(got_moves)) <= {0, 1}


def test_static_scratch_entry_point_matches_the_gpubuf_one_twice(api):
    both_entry_points(api, 4, 400, 9, seed=71, scale=synth.stress_scale(9))
    both_entry_points(api, 4, 150, 3, seed=72)  # smaller: the array still holds the first call's slots
    both_entry_points(api, 3, 90, 5, seed=73, beam_cut=3.0)
    both_entry_points(api, 5, 60, 2, seed=74)
    both_entry_points(api, 4, 120, 4, seed=75, columns=5)  # scores with a blank column, read in place
