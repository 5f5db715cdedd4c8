"""ctypes front end of the CPU oracle (oracle/libcrf_oracle.so) and, where it has
been built, of the reference's own CPU path (oracle/_ref/libopenfish_ref*.so).

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke check and by the
CPU-baseline leg of bench.py; never by the shipped package.
"""
import ctypes as C
import os
import subprocess
import tempfile

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ORACLE_SO = os.path.join(HERE, "libcrf_oracle.so")
REF_SO = os.path.join(HERE, "_ref", "libopenfish_ref.so")
REF_DEBUG_SO = os.path.join(HERE, "_ref", "libopenfish_ref_debug.so")

BEAM_WIDTH = 32
f32p = C.POINTER(C.c_float)


def build(ref=True):
    """Compile the oracle (and the reference CPU path if its tree is present)."""
    subprocess.check_call(["make", "-s", "-C", HERE, "all" if ref else os.path.join(HERE, "libcrf_oracle.so")])


class _Opt(C.Structure):
    _fields_ = [("beam_cut", C.c_float), ("blank_score", C.c_float),
                ("q_shift", C.c_float), ("q_scale", C.c_float)]


class _Dump(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in
                ("bwd", "fwd", "post", "states", "path_states", "qual_data", "base_probs", "total_probs", "beam")]


class _RefOpt(C.Structure):
    # layout of openfish_opt_t (reference include/openfish/openfish.h:29-37)
    _fields_ = [("beam_width", C.c_size_t), ("beam_cut", C.c_float), ("blank_score", C.c_float),
                ("q_shift", C.c_float), ("q_scale", C.c_float), ("temperature", C.c_float),
                ("move_pad", C.c_bool)]


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(ORACLE_SO):
            build(ref=False)
        L = C.CDLL(ORACLE_SO)
        L.ofo_crc32c.restype = C.c_uint32
        L.ofo_crc32c.argtypes = [C.c_uint32, C.c_uint32, C.c_int]
        L.ofo_set_seed_state_mask.restype = None
        L.ofo_set_seed_state_mask.argtypes = [C.c_uint32]
        L.ofo_set_scan_stay.restype = None
        L.ofo_set_scan_stay.argtypes = [C.c_float]
        L.ofo_kth_largest.restype = C.c_float
        L.ofo_kth_largest.argtypes = [f32p, C.c_int, C.c_int]
        L.ofo_log_sum_exp.restype = C.c_float
        L.ofo_log_sum_exp.argtypes = [C.c_float, C.c_float]
        for name in ("ofo_backward_scan", "ofo_forward_scan", "ofo_softmax", "ofo_decode",
                     "ofo_decode_from_tensors", "ofo_rotary_emb"):
            getattr(L, name).restype = None
        _lib = L
    return _lib


def _ptr(a):
    return a.ctypes.data_as(C.c_void_p)


def default_opt(**kw):
    o = dict(beam_cut=100.0, blank_score=2.0, q_shift=0.0, q_scale=1.0)
    o.update(kw)
    return o


def crc32c(crc, bits, nbits):
    return int(lib().ofo_crc32c(crc & 0xFFFFFFFF, bits & 0xFFFFFFFF, nbits))


def set_seed_state_mask(mask=0xFFFFFFFF):
    """test knob: seed hashes from (state & mask); a narrow mask makes sequences share hashes.
    Reset it (no argument) when done: the setting is process-wide."""
    lib().ofo_set_seed_state_mask(mask & 0xFFFFFFFF)


def set_scan_stay(stay=2.0):
    """test knob: the stay score the scans add.  The reference CPU path adds the literal 2.0 whatever
    options->blank_score says (src/decode_cpu.c:14,56); its GPU scans add blank_score
    (src/decode_hip.hip:120).  Reset it (no argument) when done: the setting is process-wide."""
    lib().ofo_set_scan_stay(C.c_float(stay))


def kth_largest(values, k):
    v = np.ascontiguousarray(values, dtype=np.float32).copy()
    return float(lib().ofo_kth_largest(v.ctypes.data_as(f32p), k, v.size))


def log_sum_exp(x, y):
    return float(lib().ofo_log_sum_exp(np.float32(x), np.float32(y)))


def scans(scores, state_len):
    """bwd, fwd(+bwd), post of every chunk; scores fp32 [T][N][4S]."""
    scores = np.ascontiguousarray(scores, dtype=np.float32)
    T, N, Cc = scores.shape
    S = 4 ** state_len
    assert Cc == 4 * S
    bwd = np.zeros((N, T + 1, S), np.float32)
    fwd = np.zeros_like(bwd)
    post = np.zeros_like(bwd)
    L = lib()
    sz = C.c_size_t
    for n in range(N):
        L.ofo_backward_scan(_ptr(scores), _ptr(bwd), sz(n), sz(T), sz(N), sz(S))
        L.ofo_forward_scan(_ptr(scores), _ptr(bwd), _ptr(fwd), sz(n), sz(T), sz(N), sz(S))
        L.ofo_softmax(_ptr(fwd), _ptr(post), sz(n), sz(T), sz(S))
    return bwd, fwd, post


def _alloc_dump(T, N, S):
    d = dict(
        bwd=np.zeros((N, T + 1, S), np.float32), fwd=np.zeros((N, T + 1, S), np.float32),
        post=np.zeros((N, T + 1, S), np.float32), states=np.zeros((N, T), np.int32),
        path_states=np.zeros((N, T), np.int32),
        qual_data=np.zeros((N, T, 4), np.float32), base_probs=np.zeros((N, T), np.float32),
        total_probs=np.zeros((N, T), np.float32),
        beam=np.zeros((N, T + 1, BEAM_WIDTH, 8), np.uint8))
    return d


def decode(scores, state_len, opt=None, nthreads=8, dump=True, C_override=None):
    """Whole CPU decode (mirrors openfish_decode_cpu).  Returns a dict with
    moves/sequence/qstring as uint8 [N][T] and, if dump, the intermediates."""
    scores = np.ascontiguousarray(scores, dtype=np.float32)
    T, N, Cc = scores.shape
    S = 4 ** state_len
    o = _Opt(**default_opt(**(opt or {})))
    out = dict(moves=np.zeros((N, T), np.uint8), sequence=np.zeros((N, T), np.uint8),
               qstring=np.zeros((N, T), np.uint8))
    dp = None
    if dump:
        d = _alloc_dump(T, N, S)
        out.update(d)
        dd = _Dump(**{k: v.ctypes.data for k, v in d.items()})
        dp = C.byref(dd)
    lib().ofo_decode(T, N, C_override or Cc, nthreads, _ptr(scores), state_len, C.byref(o),
                     _ptr(out["moves"]), _ptr(out["sequence"]), _ptr(out["qstring"]), dp)
    return out


def decode_from_tensors(scores, state_len, bwd, post, opt=None, nthreads=8, dump=True):
    """Beam search + sequence stage only, fed external bwd/post [N][T+1][S]."""
    scores = np.ascontiguousarray(scores, dtype=np.float32)
    bwd = np.ascontiguousarray(bwd, dtype=np.float32)
    post = np.ascontiguousarray(post, dtype=np.float32)
    T, N, Cc = scores.shape
    S = 4 ** state_len
    assert bwd.shape == (N, T + 1, S) and post.shape == (N, T + 1, S)
    o = _Opt(**default_opt(**(opt or {})))
    out = dict(moves=np.zeros((N, T), np.uint8), sequence=np.zeros((N, T), np.uint8),
               qstring=np.zeros((N, T), np.uint8))
    dp = None
    if dump:
        d = _alloc_dump(T, N, S)
        for k in ("bwd", "fwd", "post"):
            d.pop(k)
        out.update(d)
        dd = _Dump(**{k: v.ctypes.data for k, v in d.items()})
        dp = C.byref(dd)
    lib().ofo_decode_from_tensors(T, N, Cc, nthreads, _ptr(scores), state_len, C.byref(o), _ptr(bwd),
                                  _ptr(post), _ptr(out["moves"]), _ptr(out["sequence"]),
                                  _ptr(out["qstring"]), dp)
    return out


def rotary_emb(x, sin_buf, cos_buf, batch, seqlen, nheads, head_dim, rotary_half,
               stride_batch, stride_seq, stride_head, nthreads=4):
    """In-place fp32 rotary embedding; returns the rotated copy."""
    x = np.ascontiguousarray(x, dtype=np.float32).copy()
    s = np.ascontiguousarray(sin_buf, dtype=np.float32)
    c = np.ascontiguousarray(cos_buf, dtype=np.float32)
    lib().ofo_rotary_emb(_ptr(x), _ptr(s), _ptr(c), batch, seqlen, nheads, head_dim, rotary_half,
                         stride_batch, stride_seq, stride_head, nthreads)
    return x


def sequences(out):
    """list of (sequence str, qstring str) per chunk from a decode() result"""
    res = []
    for n in range(out["moves"].shape[0]):
        L = int(out["moves"][n].sum())
        res.append((out["sequence"][n, :L].tobytes().decode(), out["qstring"][n, :L].tobytes().decode()))
    return res


# ---- the reference's own CPU path, compiled from its sources -----------------

def have_ref():
    return os.path.exists(REF_SO)


_ref = {}


def _ref_lib(debug):
    path = REF_DEBUG_SO if debug else REF_SO
    if path not in _ref:
        L = C.CDLL(path)
        L.openfish_decode_cpu.restype = None
        L.openfish_rotary_emb_cpu.restype = None
        L.set_openfish_log_level.argtypes = [C.c_int]
        _ref[path] = L
    return _ref[path]


def ref_decode(scores, state_len, opt=None, nthreads=8, tensors=False, C_override=None):
    """openfish_decode_cpu of the compiled reference.  With tensors=True the
    -DDEBUG build is used and its blob dumps are read back."""
    scores = np.ascontiguousarray(scores, dtype=np.float32)
    T, N, Cc = scores.shape
    S = 4 ** state_len
    o = default_opt(**(opt or {}))
    ro = _RefOpt(32, o["beam_cut"], o["blank_score"], o["q_shift"], o["q_scale"], 1.0, False)
    L = _ref_lib(tensors)
    mv, sq, qs = C.c_void_p(), C.c_void_p(), C.c_void_p()
    cwd = os.getcwd()
    tmp = tempfile.mkdtemp(prefix="ofref_") if tensors else None
    try:
        if tmp:
            os.chdir(tmp)
        L.openfish_decode_cpu(T, N, C_override or Cc, nthreads, _ptr(scores), state_len, C.byref(ro),
                              C.byref(mv), C.byref(sq), C.byref(qs))
        out = {}
        for name, p in (("moves", mv), ("sequence", sq), ("qstring", qs)):
            out[name] = np.ctypeslib.as_array(C.cast(p, C.POINTER(C.c_uint8)), shape=(N, T)).copy()
        libc = C.CDLL(None)
        libc.free.argtypes = [C.c_void_p]
        for p in (mv, sq, qs):
            libc.free(p)
        if tmp:
            for name, shape in (("bwd", (N, T + 1, S)), ("fwd", (N, T + 1, S)), ("post", (N, T + 1, S)),
                                ("qual_data", (N, T, 4)), ("base_probs", (N, T)), ("total_probs", (N, T))):
                fn = {"bwd": "bwd_NTC", "fwd": "fwd_NTC", "post": "post_NTC"}.get(name, name) + ".blob"
                out[name] = np.fromfile(os.path.join(tmp, fn), dtype=np.float32).reshape(shape)
    finally:
        os.chdir(cwd)
        if tmp:
            for f in os.listdir(tmp):
                os.remove(os.path.join(tmp, f))
            os.rmdir(tmp)
    return out


def ref_rotary_emb(x, sin_buf, cos_buf, batch, seqlen, nheads, head_dim, rotary_half,
                   stride_batch, stride_seq, stride_head, nthreads=4):
    x = np.ascontiguousarray(x, dtype=np.float32).copy()
    s = np.ascontiguousarray(sin_buf, dtype=np.float32)
    c = np.ascontiguousarray(cos_buf, dtype=np.float32)
    _ref_lib(False).openfish_rotary_emb_cpu(_ptr(x), _ptr(s), _ptr(c), batch, seqlen, nheads, head_dim,
                                            rotary_half, stride_batch, stride_seq, stride_head, nthreads)
    return x
