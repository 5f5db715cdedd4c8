"""The command-line driver on the GPU: the reference's own known-answer test
(test/test.sh: decode test/data/scores.blob, diff the three result blobs)."""
import os
import subprocess

import numpy as np
import pytest

from openfish_amd import synth

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLDEN = os.path.join(ROOT, "tests", "golden")
CLI = os.path.join(ROOT, "openfish")


@pytest.fixture(scope="module")
def api():
    from openfish_amd import api as _api
    if _api.device_count() < 1:
        pytest.skip("no HIP device")
    if not os.path.exists(CLI):
        pytest.skip("command-line driver not built")
    return _api


def test_reference_fixture_through_the_cli(api, tmp_path):
    r = subprocess.run([CLI, os.path.join(GOLDEN, "ref_fixture_scores.blob"), "1", "3"], cwd=tmp_path,
                       capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr
    assert "decode completed in" in r.stderr
    for name in ("moves", "sequence", "qstring"):
        got = np.fromfile(tmp_path / (name + ".blob"), np.uint8)
        want = np.fromfile(os.path.join(GOLDEN, "ref_fixture_%s.blob" % name), np.uint8)
        assert np.array_equal(got, want), name


def test_cli_repeats_the_batch_like_the_reference_s_bench_build(api, tmp_path):
    """OPENFISH_BENCH_BATCHES=n decodes the batch n times (the reference driver's BENCH loop): same
    files as one decode, and a line with the rate"""
    env = dict(os.environ, OPENFISH_BENCH_BATCHES="5")
    r = subprocess.run([CLI, os.path.join(GOLDEN, "ref_fixture_scores.blob"), "1", "3"], cwd=tmp_path,
                       capture_output=True, text=True, timeout=120, env=env)
    assert r.returncode == 0, r.stderr
    assert "5 batches of 1 chunks" in r.stderr
    for name in ("moves", "sequence", "qstring"):
        got = np.fromfile(tmp_path / (name + ".blob"), np.uint8)
        want = np.fromfile(os.path.join(GOLDEN, "ref_fixture_%s.blob" % name), np.uint8)
        assert np.array_equal(got, want), name


def test_cli_converts_fp32_blobs_like_numpy_and_dumps_tensors(api, tmp_path):
    T, N, sl = 60, 3, 3
    rng = np.random.default_rng(8)
    s32 = (2.0 * rng.standard_normal((T, N, 256))).astype(np.float32)   # not fp16-representable
    s32[0, 0, :6] = [65503.9, 1e-8, -3.0e-5, 6.1e-5, -2049.0, 2051.0]    # near max, to zero, subnormal, ties
    s32.tofile(tmp_path / "scores32.blob")
    env = dict(os.environ, OPENFISH_DUMP_TENSORS="1")
    r = subprocess.run([CLI, "scores32.blob", str(N), str(sl), str(T)], cwd=tmp_path, env=env,
                       capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr
    # the same tensor through the library, with the fast model's calibration as the driver applies it
    gb = api.GpuBuf(T, N, sl)
    mv, sq, qs = api.openfish_decode_gpu(T, N, 256, api.upload_scores_to_hip(s32.astype(np.float16)), sl,
                                         api.DECODER_INIT(q_scale=0.97, q_shift=-1.8), gb)
    assert np.array_equal(np.fromfile(tmp_path / "moves.blob", np.uint8).reshape(N, T), mv)
    assert np.array_equal(np.fromfile(tmp_path / "sequence.blob", np.uint8).reshape(N, T), sq)
    assert np.array_equal(np.fromfile(tmp_path / "qstring.blob", np.uint8).reshape(N, T), qs)
    bwd = np.fromfile(tmp_path / "bwd_NTC.blob", np.float32).reshape(N, T + 1, 64)
    assert np.array_equal(bwd, gb.tensor("bwd_NTC"))
    for name in ("post_NTC", "qual_data", "base_probs", "total_probs"):
        assert os.path.getsize(tmp_path / (name + ".blob")) > 0


def test_cli_rejects_a_blob_of_the_wrong_size(api, tmp_path):
    np.zeros(1000, np.float32).tofile(tmp_path / "bad.blob")
    r = subprocess.run([CLI, "bad.blob", "1", "3"], cwd=tmp_path, capture_output=True, text=True, timeout=60)
    assert r.returncode != 0 and "expected T*N*C scores" in r.stderr
