"""Seeded synthetic CRF score tensors.

Every time step t has its own Philox stream keyed by (seed, t), so a tensor can
be generated in any block order, by several threads, or only for a prefix of T,
and always holds the same values.

The draw follows the five-column description of a CRF head: for every
(t, chunk, state) five values ~ N(0, sigma) with +offset on column 0 (the
blank/stay column).  The decoder consumes the four step columns only
(row layout `state*4 + dropped_base`, C = 4*4^state_len); the stay transition has
a fixed score and no column of its own (reference src/beam_search.c:211-224,
src/main.c:221).  `five_columns=True` returns the undropped tensor as well.
"""
from concurrent.futures import ThreadPoolExecutor

import numpy as np


def num_states(state_len):
    return 4 ** state_len


def _one_step(seed, t, N, S, sigma, offset, chunk_scale, five):
    rng = np.random.Generator(np.random.Philox(key=[int(seed) & 0xFFFFFFFFFFFFFFFF, int(t)]))
    g = rng.standard_normal((N, S, 5), dtype=np.float32)
    g *= np.float32(sigma)
    if chunk_scale is not None:
        g *= chunk_scale[:, None, None]
    g[:, :, 0] += np.float32(offset)
    h = g.astype(np.float16)
    four = np.ascontiguousarray(h[:, :, 1:]).reshape(N, 4 * S)
    return (four, h.reshape(N, 5 * S)) if five else (four, None)


def crf_scores(T, N, state_len, seed=1, sigma=2.0, offset=1.0, chunk_scale=None,
               five_columns=False, threads=8, out=None):
    """fp16 scores [T][N][4*S] (and optionally the [T][N][5*S] draw).

    chunk_scale: optional length-N float32 factors applied to a chunk's draw
    before the blank offset (used for the peaked / near-uniform stress mix).
    """
    S = num_states(state_len)
    if chunk_scale is not None:
        chunk_scale = np.asarray(chunk_scale, dtype=np.float32)
        assert chunk_scale.shape == (N,)
    four = out if out is not None else np.empty((T, N, 4 * S), np.float16)
    five = np.empty((T, N, 5 * S), np.float16) if five_columns else None

    def work(t):
        a, b = _one_step(seed, t, N, S, sigma, offset, chunk_scale, five_columns)
        four[t] = a
        if five_columns:
            five[t] = b

    if threads > 1 and T > 1:
        with ThreadPoolExecutor(threads) as ex:
            list(ex.map(work, range(T)))
    else:
        for t in range(T):
            work(t)
    return (four, five) if five_columns else four


def stress_scale(N, peaked=6.0, flat=0.2):
    """even chunks sharply peaked, odd chunks near-uniform"""
    s = np.full(N, flat, np.float32)
    s[0::2] = peaked
    return s


def rotary_tables(seqlen, rotary_half, base=10000.0):
    """fp32 sin/cos tables [seqlen][rotary_half]"""
    inv = 1.0 / (base ** (np.arange(rotary_half, dtype=np.float64) / rotary_half))
    ang = np.arange(seqlen, dtype=np.float64)[:, None] * inv[None, :]
    return np.sin(ang).astype(np.float32), np.cos(ang).astype(np.float32)
