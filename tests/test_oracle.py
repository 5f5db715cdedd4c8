"""Pins the CPU oracle (oracle/crf_oracle.c): golden vectors written by the
compiled reference, the reference's own in-repo fixture, closed forms and brute
force.  No GPU needed."""
import glob
import itertools
import os

import numpy as np
import pytest

from openfish_amd import synth
from oracle import crf_oracle as O

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")
CASES = sorted(os.path.basename(p)[:-4] for p in glob.glob(os.path.join(GOLDEN, "*.npz")))


def bits(a):
    return a.view(np.uint32) if a.dtype == np.float32 else a


def load(name):
    z = np.load(os.path.join(GOLDEN, name + ".npz"))
    bc, bl, qs, qc = [float(v) for v in z["opt"]]
    return z, int(z["state_len"]), dict(beam_cut=bc, blank_score=bl, q_shift=qs, q_scale=qc)


# ---- helpers with textbook answers ------------------------------------------

def test_crc32c_check_value():
    # CRC-32C("123456789") = 0xE3069283 with the usual ~0 init and final inversion
    crc = 0xFFFFFFFF
    for ch in b"123456789":
        crc = O.crc32c(crc, ch, 8)
    assert crc ^ 0xFFFFFFFF == 0xE3069283


def test_crc32c_bitwise_composition():
    # feeding 32 bits at once equals feeding them two at a time, LSB first
    rng = np.random.default_rng(0)
    for _ in range(50):
        crc, word = int(rng.integers(0, 2 ** 32)), int(rng.integers(0, 2 ** 32))
        step = crc
        for k in range(16):
            step = O.crc32c(step, (word >> (2 * k)) & 3, 2)
        assert step == O.crc32c(crc, word, 32)


@pytest.mark.parametrize("n", [33, 64, 256, 1024])
def test_kth_largest_is_order_statistic(n):
    rng = np.random.default_rng(n)
    for trial in range(20):
        v = rng.standard_normal(n).astype(np.float32)
        if trial % 3 == 1:
            v = np.round(v * 2) / 2  # many ties
        if trial % 3 == 2:
            v[:] = v[0]              # all equal
        assert O.kth_largest(v, 31) == np.sort(v)[::-1][31]


def test_log_sum_exp_closed_form():
    rng = np.random.default_rng(1)
    for _ in range(200):
        x, y = (rng.standard_normal(2) * 10).astype(np.float32)
        got = O.log_sum_exp(x, y)
        gap = abs(float(np.float32(x) - np.float32(y)))
        want = max(x, y) + (np.log1p(np.exp(-gap)) if gap < 17.0 else 0.0)
        assert got == np.float32(want)
    assert O.log_sum_exp(3.0, 3.0 - 17.0) == np.float32(3.0)      # cut-off reached: no correction
    assert O.log_sum_exp(0.0, 0.0) == np.float32(np.log(2.0))


# ---- scans: closed form, invariants, brute force ----------------------------

@pytest.mark.parametrize("state_len", [1, 2, 3])
def test_scans_constant_scores_closed_form(state_len):
    T, N, S = 40, 2, 4 ** state_len
    c = 0.75
    sc = np.full((T, N, 4 * S), c, np.float32)
    bwd, fwd, post = O.scans(sc, state_len)
    per_step = np.log(np.exp(2.0) + 4 * np.exp(c))
    want = (T - np.arange(T + 1)) * per_step
    np.testing.assert_allclose(bwd, np.broadcast_to(want[None, :, None], bwd.shape), rtol=2e-6)
    np.testing.assert_allclose(fwd, T * per_step, rtol=2e-6)
    np.testing.assert_allclose(post, 1.0 / S, rtol=1e-5)


def transition_matrices(sc64, state_len, stay=2.0):
    """dense per-step matrices from the k-mer definition: from k-mer p a step
    appends base b giving s = ((p<<2) & mask) | b, scored by entry s*4 + (leading
    base of p); staying in p scores `stay` (2.0 on the reference CPU path)"""
    T, C = sc64.shape
    S = 4 ** state_len
    M = np.zeros((T, S, S))
    for p in range(S):
        lead = p >> (2 * (state_len - 1))
        for b in range(4):
            s = ((p << 2) & (S - 1)) | b
            M[:, p, s] += np.exp(sc64[:, s * 4 + lead])
        M[:, p, p] += np.exp(stay)
    return M


@pytest.mark.parametrize("state_len,T", [(1, 6), (2, 9), (3, 12)])
def test_scans_against_dense_matrix_products(state_len, T):
    N, S = 2, 4 ** state_len
    s32 = synth.crf_scores(T, N, state_len, seed=3).astype(np.float32)
    bwd, fwd, post = O.scans(s32, state_len)
    for n in range(N):
        M = transition_matrices(s32[:, n, :].astype(np.float64), state_len)
        beta = np.ones(S)
        want_b = [np.zeros(S)]
        for t in range(T - 1, -1, -1):
            beta = M[t] @ beta
            want_b.append(np.log(beta))
        want_b = np.array(want_b[::-1])
        np.testing.assert_allclose(bwd[n], want_b, rtol=1e-5, atol=1e-5)
        alpha = np.ones(S)
        want_f = [np.zeros(S)]
        for t in range(T):
            alpha = alpha @ M[t]
            want_f.append(np.log(alpha))
        want_f = np.array(want_f)
        np.testing.assert_allclose(fwd[n], want_f + want_b, rtol=1e-5, atol=1e-5)
        joint = np.exp(want_f + want_b - (want_f + want_b).max(axis=1, keepdims=True))
        np.testing.assert_allclose(post[n], joint / joint.sum(axis=1, keepdims=True), rtol=1e-4, atol=1e-7)


@pytest.mark.parametrize("stay", [0.5, -1.5, 5.0])
def test_scan_stay_knob_against_closed_form_and_dense_products(stay):
    """the oracle's scans with another stay score than the CPU path's 2.0 (what the reference's GPU
    scans do with options->blank_score, src/decode_hip.hip:120): closed form on constant scores,
    and dense transition-matrix products with e^stay on the diagonal"""
    O.set_scan_stay(stay)
    try:
        T, N, sl, c = 40, 2, 3, -0.25
        S = 4 ** sl
        bwd, fwd, post = O.scans(np.full((T, N, 4 * S), c, np.float32), sl)
        per_step = np.log(np.exp(stay) + 4 * np.exp(c))
        want = (T - np.arange(T + 1)) * per_step
        np.testing.assert_allclose(bwd, np.broadcast_to(want[None, :, None], bwd.shape), rtol=2e-6, atol=1e-6)
        np.testing.assert_allclose(fwd, T * per_step, rtol=2e-6)
        np.testing.assert_allclose(post, 1.0 / S, rtol=1e-5)
        T = 12
        s32 = synth.crf_scores(T, N, sl, seed=5).astype(np.float32)
        bwd, fwd, post = O.scans(s32, sl)
        for n in range(N):
            M = transition_matrices(s32[:, n, :].astype(np.float64), sl, stay)
            beta = np.ones(S)
            want_b = [np.zeros(S)]
            for t in range(T - 1, -1, -1):
                beta = M[t] @ beta
                want_b.append(np.log(beta))
            want_b = np.array(want_b[::-1])
            np.testing.assert_allclose(bwd[n], want_b, rtol=1e-5, atol=1e-5)
            alpha = np.ones(S)
            want_f = [np.zeros(S)]
            for t in range(T):
                alpha = alpha @ M[t]
                want_f.append(np.log(alpha))
            want_f = np.array(want_f)
            np.testing.assert_allclose(fwd[n], want_f + want_b, rtol=1e-5, atol=1e-5)
    finally:
        O.set_scan_stay()
    # back at the CPU path's literal: the default scans are the golden-pinned ones again
    bwd2, _, _ = O.scans(np.full((8, 1, 4 * 64), 0.5, np.float32), 3)
    np.testing.assert_allclose(bwd2[0, 0, 0], 8 * np.log(np.exp(2.0) + 4 * np.exp(0.5)), rtol=2e-6)


def test_state_len1_brute_force_paths():
    # enumerate every state path for S=4 and sum path weights directly
    T, state_len, S = 4, 1, 4
    s32 = synth.crf_scores(T, 1, state_len, seed=5).astype(np.float32)
    sc = s32[:, 0, :].astype(np.float64)
    bwd, _, _ = O.scans(s32, state_len)
    for start in range(S):
        total = 0.0
        for path in itertools.product(range(S), repeat=T):
            w, p = 1.0, start
            for t, s in enumerate(path):
                w *= np.exp(sc[t, s * 4 + p]) + (np.exp(2.0) if s == p else 0.0)
                p = s
            total += w
        assert np.isclose(bwd[0, 0, start], np.log(total), rtol=1e-5)


def test_posterior_rows_sum_to_one_and_logz_is_constant():
    T, N, sl = 200, 2, 3
    s32 = synth.crf_scores(T, N, sl, seed=9).astype(np.float32)
    bwd, fwd, post = O.scans(s32, sl)
    assert np.all(bwd[:, T, :] == 0.0)
    np.testing.assert_allclose(post.sum(axis=2), 1.0, rtol=1e-5)
    m = fwd.max(axis=2, keepdims=True)
    logz = (m + np.log(np.exp(fwd - m).sum(axis=2, keepdims=True)))[..., 0]
    np.testing.assert_allclose(logz, np.broadcast_to(logz[:, :1], logz.shape), rtol=1e-5)


# ---- golden vectors -----------------------------------------------------------

def test_reference_in_repo_fixture():
    sc = np.fromfile(os.path.join(GOLDEN, "ref_fixture_scores.blob"), np.float32).reshape(1666, 1, 256)
    out = O.decode(sc, 3, dict(q_scale=0.97, q_shift=-1.8), nthreads=1)
    for k in ("moves", "sequence", "qstring"):
        want = np.fromfile(os.path.join(GOLDEN, "ref_fixture_%s.blob" % k), np.uint8).reshape(1, 1666)
        assert np.array_equal(out[k], want), k
    assert O.sequences(out)[0][0] == "G" * 32


@pytest.mark.parametrize("name", CASES)
def test_oracle_equals_reference_golden(name):
    z, sl, opt = load(name)
    out = O.decode(z["scores"].astype(np.float32), sl, opt, nthreads=2)
    for k in ("bwd", "fwd", "post", "moves", "sequence", "qstring", "qual_data", "base_probs", "total_probs"):
        assert np.array_equal(bits(out[k]), bits(z[k])), (name, k)


@pytest.mark.parametrize("name", CASES)
def test_beam_stage_from_golden_tensors(name):
    z, sl, opt = load(name)
    out = O.decode_from_tensors(z["scores"].astype(np.float32), sl, z["bwd"], z["post"], opt, nthreads=2)
    for k in ("moves", "sequence", "qstring", "qual_data"):
        assert np.array_equal(bits(out[k]), bits(z[k])), (name, k)


def test_thread_count_does_not_change_results():
    s32 = synth.crf_scores(120, 7, 3, seed=21).astype(np.float32)
    a = O.decode(s32, 3, nthreads=1)
    b = O.decode(s32, 3, nthreads=5)
    for k in a:
        assert np.array_equal(bits(a[k]), bits(b[k])), k


@pytest.mark.skipif(not O.have_ref(), reason="compiled reference (oracle/_ref) not built here")
@pytest.mark.parametrize("state_len,T,N,stress", [(3, 500, 6, False), (3, 500, 6, True), (4, 300, 3, True),
                                                   (5, 80, 2, False), (2, 100, 4, True)])
def test_oracle_equals_compiled_reference_live(state_len, T, N, stress):
    scale = synth.stress_scale(N) if stress else None
    s32 = synth.crf_scores(T, N, state_len, seed=100 + T, chunk_scale=scale).astype(np.float32)
    opt = dict(q_scale=0.95, q_shift=-0.2)
    a = O.decode(s32, state_len, opt, nthreads=3)
    b = O.ref_decode(s32, state_len, opt, nthreads=3, tensors=True)
    for k in b:
        assert np.array_equal(bits(a[k]), bits(b[k])), k


# ---- rotary embedding ---------------------------------------------------------

def rotary_case(batch=3, seqlen=17, nheads=4, head_dim=16, rotary_half=8, seed=2):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((batch, seqlen, nheads, head_dim)).astype(np.float32)
    sn, cs = synth.rotary_tables(seqlen, rotary_half)
    strides = (seqlen * nheads * head_dim, nheads * head_dim, head_dim)
    return x, sn, cs, (batch, seqlen, nheads, head_dim, rotary_half) + strides


def test_rotary_is_a_plane_rotation():
    x, sn, cs, dims = rotary_case()
    y = O.rotary_emb(x, sn, cs, *dims).reshape(x.shape)
    h = dims[4]
    x0, x1 = x[..., :h], x[..., h:2 * h]
    c, s = cs[None, :, None, :], sn[None, :, None, :]
    np.testing.assert_array_equal(y[..., :h], x0 * c - x1 * s)
    np.testing.assert_array_equal(y[..., h:2 * h], x0 * s + x1 * c)
    np.testing.assert_array_equal(y[..., 2 * h:], x[..., 2 * h:])          # untouched tail
    np.testing.assert_allclose((y[..., :2 * h] ** 2).sum(-1), (x[..., :2 * h] ** 2).sum(-1), rtol=1e-5)


@pytest.mark.skipif(not O.have_ref(), reason="compiled reference (oracle/_ref) not built here")
def test_rotary_equals_compiled_reference():
    x, sn, cs, dims = rotary_case(batch=5, seqlen=33, nheads=8, head_dim=64, rotary_half=32)
    a = O.rotary_emb(x, sn, cs, *dims)
    b = O.ref_rotary_emb(x, sn, cs, *dims)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
