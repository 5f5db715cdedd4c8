"""Python mirror of the openfish C API, bound with ctypes to
openfish_amd/libopenfish_amd.so (the same objects as lib/libopenfish.a).

The functions keep the C names and argument meaning (include/openfish/openfish.h,
include/openfish/openfish_amd.h).  There is no fallback of any kind: if the
shared library has not been built the import of this module fails, and any
device error makes the C library print a message and exit the process, as the
reference library does.
"""
import ctypes as C
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libopenfish_amd.so")

if not os.path.exists(LIB_PATH):
    raise ImportError(
        "%s is missing: build it with `make` at the repository root "
        "(or __graft_entry__.build()); there is no CPU fallback" % LIB_PATH)

_L = C.CDLL(LIB_PATH)

STAGES = ("bwd", "fwd_post", "beam", "sequence", "total", "scan", "path_sums")
# enum openfish_amd_scan_mode
SCAN_TWO_TIER, SCAN_PRECISE, SCAN_FAST = 0, 1, 2
SCAN_MODES = {"two_tier": SCAN_TWO_TIER, "precise": SCAN_PRECISE, "fast": SCAN_FAST}


class openfish_opt_t(C.Structure):
    """reference include/openfish/openfish.h:29-37"""
    _fields_ = [("beam_width", C.c_size_t), ("beam_cut", C.c_float), ("blank_score", C.c_float),
                ("q_shift", C.c_float), ("q_scale", C.c_float), ("temperature", C.c_float),
                ("move_pad", C.c_bool)]


class openfish_gpubuf_t(C.Structure):
    """reference include/openfish/openfish.h:16-27"""
    _fields_ = [("bwd_NTC", C.c_void_p), ("post_NTC", C.c_void_p), ("moves", C.c_void_p),
                ("sequence", C.c_void_p), ("qstring", C.c_void_p), ("beam_vector", C.c_void_p),
                ("states", C.c_void_p), ("qual_data", C.c_void_p), ("base_probs", C.c_void_p),
                ("total_probs", C.c_void_p)]


def DECODER_INIT(**kw):
    """{32, 100.0, 2.0, 0.0, 1.0, 1.0, false} with keyword overrides"""
    o = openfish_opt_t(32, 100.0, 2.0, 0.0, 1.0, 1.0, False)
    for k, v in kw.items():
        setattr(o, k, v)
    return o


_vp, _i, _f, _sz = C.c_void_p, C.c_int, C.c_float, C.c_size_t
_optp, _bufp = C.POINTER(openfish_opt_t), C.POINTER(openfish_gpubuf_t)
_pp = C.POINTER(C.c_void_p)

_SIGS = {
    "openfish_gpubuf_init": (_bufp, [_i, _i, _i]),
    "openfish_gpubuf_free": (None, [_bufp]),
    "openfish_decode_gpu": (None, [_i, _i, _i, _vp, _i, _optp, _bufp, _pp, _pp, _pp]),
    "openfish_rotary_emb_gpu": (None, [_vp, _vp, _vp] + [_i] * 8),
    "openfish_decode_cpu": (None, [_i, _i, _i, _i, _vp, _i, _optp, _pp, _pp, _pp]),
    "openfish_rotary_emb_cpu": (None, [_vp, _vp, _vp] + [_i] * 9),
    "get_openfish_log_level": (_i, []),
    "set_openfish_log_level": (None, [_i]),
    "set_device_hip": (None, [_i]),
    "upload_scores_to_hip": (_vp, [_i, _i, _i, _vp]),
    "free_scores_hip": (None, [_vp]),
    "write_gpubuf_hip": (None, [C.c_uint64, C.c_uint64, _i, _bufp]),
    "openfish_amd_malloc": (_vp, [_sz]),
    "openfish_amd_free": (None, [_vp]),
    "openfish_amd_memcpy_h2d": (None, [_vp, _vp, _sz]),
    "openfish_amd_memcpy_d2h": (None, [_vp, _vp, _sz]),
    "openfish_amd_memset": (None, [_vp, _i, _sz]),
    "openfish_amd_sync": (None, []),
    "openfish_amd_copy": (None, [_vp, _vp, _sz]),
    "openfish_amd_device_count": (_i, []),
    "openfish_amd_bwd_scan": (None, [_i, _i, _i, _vp, _i, _f, _i, _vp]),
    "openfish_amd_fwd_post_scan": (None, [_i, _i, _i, _vp, _i, _f, _i, _vp, _vp]),
    "openfish_amd_scan_posterior": (None, [_i, _i, _i, _vp, _i, _f, _i, _vp, _vp]),
    "openfish_amd_gpubuf_set_split_scans": (None, [_bufp, _i]),
    "openfish_amd_beam_search": (None, [_i, _i, _i, _vp, _i, _optp, _vp, _bufp]),
    "openfish_amd_beam_search_static_prepare": (None, []),
    "openfish_amd_beam_search_static": (None, [_i, _i, _i, _vp, _i, _optp, _vp, _vp, _vp, _vp]),
    "openfish_amd_device_free_bytes": (_sz, []),
    "openfish_amd_sequence": (None, [_i, _i, _i, _optp, _vp, _bufp]),
    "openfish_amd_decode_enqueue": (None, [_i, _i, _i, _vp, _i, _optp, _bufp]),
    "openfish_amd_decode_wait": (None, [_bufp, _pp, _pp, _pp]),
    "openfish_amd_decode_from_tensors": (None, [_i, _i, _i, _vp, _i, _optp, _vp, _vp, _bufp, _pp, _pp, _pp]),
    "openfish_amd_last_timings": (_i, [_bufp, C.POINTER(C.c_float), _i]),
    "openfish_amd_gpubuf_set_debug_flags": (None, [_bufp, _i]),
    "openfish_amd_gpubuf_set_scan_mode": (None, [_bufp, _i]),
    "openfish_amd_gpubuf_set_scan_states_per_lane": (None, [_bufp, _i]),
    "openfish_amd_lse_table": (None, [C.POINTER(C.c_double)]),
    "openfish_amd_phred_table": (None, [_f, _f, C.POINTER(C.c_float)]),
    "openfish_amd_probe_hw_math": (None, [C.POINTER(C.c_double), C.POINTER(C.c_uint)]),
    "openfish_amd_version": (C.c_char_p, []),
}

EXPORTS = tuple(_SIGS)

for _name, (_res, _args) in _SIGS.items():
    _fn = getattr(_L, _name)  # AttributeError here means the library lacks a declared symbol
    _fn.restype = _res
    _fn.argtypes = _args

_libc = C.CDLL(None)
_libc.free.argtypes = [C.c_void_p]


def lib():
    return _L


def device_count():
    return int(_L.openfish_amd_device_count())


class DeviceBuffer:
    """a device allocation owned by Python"""

    def __init__(self, nbytes):
        self.nbytes = int(nbytes)
        self.ptr = _L.openfish_amd_malloc(self.nbytes)

    @classmethod
    def from_host(cls, array):
        a = np.ascontiguousarray(array)
        b = cls(a.nbytes)
        _L.openfish_amd_memcpy_h2d(b.ptr, a.ctypes.data, a.nbytes)
        return b

    def to_host(self, dtype, shape):
        out = np.empty(shape, dtype)
        assert out.nbytes <= self.nbytes
        _L.openfish_amd_memcpy_d2h(out.ctypes.data, self.ptr, out.nbytes)
        return out

    def fill(self, byte):
        _L.openfish_amd_memset(self.ptr, byte, self.nbytes)

    def free(self):
        if self.ptr:
            _L.openfish_amd_free(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def _device_to_host(ptr, dtype, shape):
    out = np.empty(shape, dtype)
    _L.openfish_amd_memcpy_d2h(out.ctypes.data, ptr, out.nbytes)
    return out


def _take(ptr, N, T):
    """copy one malloc'd [N][T] byte buffer returned by the C API and free it"""
    a = np.ctypeslib.as_array(C.cast(ptr, C.POINTER(C.c_uint8)), shape=(N, T)).copy()
    _libc.free(ptr)
    return a


class GpuBuf:
    """openfish_gpubuf_init / openfish_gpubuf_free"""

    def __init__(self, T, N, state_len):
        self.T, self.N, self.state_len = T, N, state_len
        self.S = 4 ** state_len
        self.handle = _L.openfish_gpubuf_init(T, N, state_len)

    def free(self):
        if self.handle:
            _L.openfish_gpubuf_free(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass

    def tensor(self, name, T=None, N=None):
        """host copy of one device tensor of the gpubuf"""
        T = T or self.T
        N = N or self.N
        f = self.handle.contents
        shapes = {
            "bwd_NTC": (np.float32, (N, T + 1, self.S)), "post_NTC": (np.float32, (N, T + 1, self.S)),
            "moves": (np.uint8, (N, T)), "sequence": (np.uint8, (N, T)), "qstring": (np.uint8, (N, T)),
            "states": (np.int32, (N, T)), "qual_data": (np.float32, (N, T, 4)),
            "base_probs": (np.float32, (N, T)), "total_probs": (np.float32, (N, T)),
            "beam_vector": (np.uint16, (N, T + 1, 32)),
        }
        dt, shp = shapes[name]
        return _device_to_host(getattr(f, name), dt, shp)

    def set_scan_mode(self, mode):
        """mode: SCAN_TWO_TIER (default), SCAN_PRECISE or SCAN_FAST, or their names"""
        _L.openfish_amd_gpubuf_set_scan_mode(self.handle, SCAN_MODES.get(mode, mode))

    def set_split_scans(self, split):
        """True: backward scan, then forward scan + posterior beside the beam search; False: both
        scans as one kernel; None: the library chooses per call (the default)"""
        _L.openfish_amd_gpubuf_set_split_scans(self.handle, -1 if split is None else (1 if split else 0))

    def set_scan_states_per_lane(self, spl):
        _L.openfish_amd_gpubuf_set_scan_states_per_lane(self.handle, int(spl))

    def set_debug_flags(self, flags):
        _L.openfish_amd_gpubuf_set_debug_flags(self.handle, int(flags))

    def timings(self):
        """device-side milliseconds of the stages of the last openfish_decode_gpu call"""
        ms = (C.c_float * len(STAGES))()
        n = _L.openfish_amd_last_timings(self.handle, ms, len(STAGES))
        return {STAGES[k]: float(ms[k]) for k in range(n)}


def openfish_decode_gpu(T, N, Cc, scores_dev, state_len, options, gpubuf):
    """returns (moves, sequence, qstring) as uint8 [N][T] host arrays"""
    mv, sq, qs = C.c_void_p(), C.c_void_p(), C.c_void_p()
    _L.openfish_decode_gpu(T, N, Cc, _ptr(scores_dev), state_len, C.byref(options), gpubuf.handle,
                           C.byref(mv), C.byref(sq), C.byref(qs))
    return _take(mv, N, T), _take(sq, N, T), _take(qs, N, T)


def openfish_decode_gpu_discard(T, N, Cc, scores_dev, state_len, options, gpubuf):
    """the same C call, results freed without a copy into numpy (what a timing loop wants: the
    call and the caller's three free()s, nothing of this wrapper)"""
    mv, sq, qs = C.c_void_p(), C.c_void_p(), C.c_void_p()
    _L.openfish_decode_gpu(T, N, Cc, _ptr(scores_dev), state_len, C.byref(options), gpubuf.handle,
                           C.byref(mv), C.byref(sq), C.byref(qs))
    _libc.free(mv)
    _libc.free(sq)
    _libc.free(qs)


def openfish_amd_decode_enqueue(T, N, Cc, scores_dev, state_len, options, gpubuf):
    """queue one decode on the gpubuf and return at once; scores_dev must stay alive until the wait"""
    _L.openfish_amd_decode_enqueue(T, N, Cc, _ptr(scores_dev), state_len, C.byref(options), gpubuf.handle)
    gpubuf._pending_shape = (N, T)


def openfish_amd_decode_wait(gpubuf, copy=True):
    """(moves, sequence, qstring) of the enqueued decode as uint8 [N, T] arrays (copies of the
    library's pinned buffer); copy=False only waits (timing loops)"""
    N, T = gpubuf._pending_shape
    mv, sq, qs = C.c_void_p(), C.c_void_p(), C.c_void_p()
    _L.openfish_amd_decode_wait(gpubuf.handle, C.byref(mv), C.byref(sq), C.byref(qs))
    if not copy:
        return None
    out = []
    for p in (mv, sq, qs):
        buf = (C.c_uint8 * (N * T)).from_address(p.value)
        out.append(np.frombuffer(buf, np.uint8).reshape(N, T).copy())
    return tuple(out)


def openfish_amd_decode_from_tensors(T, N, Cc, scores_dev, state_len, options, bwd_dev, post_dev, gpubuf):
    mv, sq, qs = C.c_void_p(), C.c_void_p(), C.c_void_p()
    _L.openfish_amd_decode_from_tensors(T, N, Cc, _ptr(scores_dev), state_len, C.byref(options),
                                        _ptr(bwd_dev), _ptr(post_dev), gpubuf.handle,
                                        C.byref(mv), C.byref(sq), C.byref(qs))
    return _take(mv, N, T), _take(sq, N, T), _take(qs, N, T)


def openfish_amd_bwd_scan(T, N, Cc, scores_dev, state_len, stay_score, bwd_dev, scan_mode=SCAN_TWO_TIER):
    _L.openfish_amd_bwd_scan(T, N, Cc, _ptr(scores_dev), state_len, stay_score, SCAN_MODES.get(scan_mode, scan_mode),
                             _ptr(bwd_dev))


def openfish_amd_fwd_post_scan(T, N, Cc, scores_dev, state_len, stay_score, bwd_dev, post_dev,
                               scan_mode=SCAN_TWO_TIER):
    _L.openfish_amd_fwd_post_scan(T, N, Cc, _ptr(scores_dev), state_len, stay_score,
                                  SCAN_MODES.get(scan_mode, scan_mode), _ptr(bwd_dev), _ptr(post_dev))


def openfish_amd_scan_posterior(T, N, Cc, scores_dev, state_len, stay_score, bwd_dev, post_dev,
                                scan_mode=SCAN_TWO_TIER):
    _L.openfish_amd_scan_posterior(T, N, Cc, _ptr(scores_dev), state_len, stay_score,
                                   SCAN_MODES.get(scan_mode, scan_mode), _ptr(bwd_dev), _ptr(post_dev))


def openfish_amd_beam_search(T, N, Cc, scores_dev, state_len, options, bwd_dev, gpubuf):
    _L.openfish_amd_beam_search(T, N, Cc, _ptr(scores_dev), state_len, C.byref(options), _ptr(bwd_dev), gpubuf.handle)


def openfish_amd_beam_search_static_prepare():
    """set up the library's static scratch array on the current device (once; blocking)"""
    _L.openfish_amd_beam_search_static_prepare()


def openfish_amd_beam_search_static(T, N, Cc, scores_dev, state_len, options, bwd_dev, states_dev, moves_dev,
                                    stream=None):
    """the beam search on the library's static scratch array: launches on `stream` and returns;
    allocates nothing, copies nothing, waits for nothing (openfish_amd_sync() before reading results)"""
    _L.openfish_amd_beam_search_static(T, N, Cc, _ptr(scores_dev), state_len, C.byref(options), _ptr(bwd_dev),
                                       _ptr(states_dev), _ptr(moves_dev), stream)


def device_free_bytes():
    return int(_L.openfish_amd_device_free_bytes())


def openfish_amd_sequence(T, N, state_len, options, post_dev, gpubuf):
    _L.openfish_amd_sequence(T, N, state_len, C.byref(options), _ptr(post_dev), gpubuf.handle)


def openfish_rotary_emb_gpu(x_dev, sin_dev, cos_dev, batch_size, seqlen, nheads, head_dim, rotary_half,
                            stride_batch, stride_seq, stride_head):
    _L.openfish_rotary_emb_gpu(_ptr(x_dev), _ptr(sin_dev), _ptr(cos_dev), batch_size, seqlen, nheads,
                               head_dim, rotary_half, stride_batch, stride_seq, stride_head)


def upload_scores_to_hip(scores_half):
    """host fp16 [T][N][C] -> DeviceBuffer (reference upload_scores_to_hip)"""
    a = np.ascontiguousarray(scores_half, dtype=np.float16)
    return DeviceBuffer.from_host(a)


def phred_table(q_scale, q_shift):
    thr = (C.c_float * 49)()
    _L.openfish_amd_phred_table(q_scale, q_shift, thr)
    return np.array(thr[:], dtype=np.float32)


def probe_hw_math():
    """(errors in units of 2^-24: exp on [-160,0], log on [1,2), [2,4), [4,5.01]; identity bits)"""
    err = (C.c_double * 4)()
    ident = C.c_uint(0)
    _L.openfish_amd_probe_hw_math(err, C.byref(ident))
    return [float(x) for x in err], int(ident.value)


def lse_table():
    """[68][9] coefficients of log(1 + e^-gap) per quarter-unit cell"""
    tab = (C.c_double * (68 * 9))()
    _L.openfish_amd_lse_table(tab)
    return np.array(tab[:], dtype=np.float64).reshape(68, 9)


def _ptr(x):
    if isinstance(x, DeviceBuffer):
        return x.ptr
    return x
