"""The C-ABI library without a GPU: it loads, exports every function the headers
declare, keeps the reference struct layouts, and its host-side logic (phred
thresholds, argument checks, exit-on-error convention) behaves as documented."""
import ctypes as C
import os
import re
import subprocess
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
INCLUDE = os.path.join(ROOT, "include", "openfish")


def declared_functions():
    names = set()
    for header in ("openfish.h", "openfish_error.h", "openfish_amd.h"):
        text = open(os.path.join(INCLUDE, header)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        text = re.sub(r"^\s*#.*?(?<!\\)$", "", text, flags=re.M)
        for m in re.finditer(r"\b([A-Za-z_][A-Za-z0-9_]*)\s*\([^;{}()]*\)\s*(?:__attribute__\(\(.*?\)\)\s*)?;", text, flags=re.S):
            names.add(m.group(1))
    return sorted(names - {"__attribute__", "format", "defined"})


def test_library_loads_and_exports_every_declared_symbol():
    from openfish_amd import api
    names = declared_functions()
    assert len(names) >= 25, names
    for required in ("openfish_decode_gpu", "openfish_gpubuf_init", "openfish_gpubuf_free",
                     "openfish_rotary_emb_gpu", "openfish_decode_cpu", "openfish_rotary_emb_cpu",
                     "get_openfish_log_level", "set_openfish_log_level", "set_device_hip",
                     "upload_scores_to_hip", "free_scores_hip", "write_gpubuf_hip"):
        assert required in names
    for n in names:
        assert hasattr(api.lib(), n), "library lacks %s" % n


def test_static_library_has_the_public_symbols():
    path = os.path.join(ROOT, "lib", "libopenfish.a")
    if not os.path.exists(path):
        pytest.skip("lib/libopenfish.a not built")
    out = subprocess.run(["nm", "-g", "--defined-only", path], capture_output=True, text=True).stdout
    for n in ("openfish_decode_gpu", "openfish_gpubuf_init", "openfish_gpubuf_free", "openfish_rotary_emb_gpu",
              "get_openfish_log_level", "set_openfish_log_level"):
        assert re.search(r"\bT %s\b" % n, out), n


def test_struct_layouts_match_the_reference_header():
    from openfish_amd import api
    # openfish_opt_t: size_t + 5 floats + bool, padded to 32 bytes; gpubuf: ten pointers
    assert C.sizeof(api.openfish_opt_t) == 32
    assert api.openfish_opt_t.beam_cut.offset == 8 and api.openfish_opt_t.move_pad.offset == 28
    assert C.sizeof(api.openfish_gpubuf_t) == 80
    o = api.DECODER_INIT()
    assert (o.beam_width, o.beam_cut, o.blank_score, o.q_shift, o.q_scale, o.temperature, o.move_pad) == \
        (32, 100.0, 2.0, 0.0, 1.0, 1.0, False)


def test_log_level_roundtrip():
    from openfish_amd import api
    L = api.lib()
    assert L.get_openfish_log_level() == 4  # OPENFISH_LOG_VERB, the reference default
    L.set_openfish_log_level(2)
    assert L.get_openfish_log_level() == 2
    L.set_openfish_log_level(4)


def phred_direct(x, scale, shift, log10f):
    f32 = np.float32
    v = f32(-10.0) * f32(log10f(float(x)))
    q = f32(v * f32(scale))
    q = f32(q + f32(shift))
    q = min(q, f32(50.0))
    q = max(q, f32(1.0))
    return int(f32(33.5) + q)


@pytest.mark.parametrize("scale,shift", [(1.0, 0.0), (0.97, -1.8), (0.95, -0.2), (0.95, 0.5), (1.3, 4.0)])
def test_phred_thresholds_reproduce_libm_characters(scale, shift):
    from openfish_amd import api
    libm = C.CDLL("libm.so.6")
    libm.log10f.restype = C.c_float
    libm.log10f.argtypes = [C.c_float]
    thr = api.phred_table(scale, shift)
    assert np.all(np.diff(thr) >= 0)
    rng = np.random.default_rng(5)
    xs = [rng.random(3000).astype(np.float32), (10.0 ** (-6 * rng.random(3000))).astype(np.float32),
          np.array([0.0, 1.0, 1e-30, 1e-45], np.float32)]
    bits = thr[thr <= 1.0].view(np.uint32).astype(np.int64)
    for d in range(-2, 3):  # the floats right at every threshold
        xs.append(np.clip(bits + d, 0, 0x3F800000).astype(np.uint32).view(np.float32))
    for x in np.concatenate(xs):
        assert 83 - int((x >= thr).sum()) == phred_direct(x, scale, shift, libm.log10f), float(x)


def run_snippet(code):
    return subprocess.run([sys.executable, "-c", "import sys; sys.path.insert(0, %r)\n%s" % (ROOT, code)],
                          capture_output=True, text=True, timeout=120)


def test_wrong_channel_count_exits_with_message():
    # a channel count that is neither 4*S nor 5*S: message + exit, no GPU touched
    r = run_snippet("import ctypes as C\nfrom openfish_amd import api\n"
                    "o = api.DECODER_INIT()\nmv, sq, qs = C.c_void_p(), C.c_void_p(), C.c_void_p()\n"
                    "api.lib().openfish_decode_gpu(10, 2, 300, 4096, 3, C.byref(o), None, C.byref(mv), C.byref(sq), C.byref(qs))\n"
                    "print('survived')")
    assert r.returncode != 0 and "survived" not in r.stdout
    assert "C must be 4 * 4^state_len" in r.stderr


def test_unsupported_state_len_exits_with_message():
    r = run_snippet("from openfish_amd import api\napi.lib().openfish_gpubuf_init(100, 4, 2)\nprint('survived')")
    assert r.returncode != 0 and "survived" not in r.stdout
    assert "state_len must be 3, 4 or 5" in r.stderr


def test_cpu_entry_points_exit_loudly():
    r = run_snippet("from openfish_amd import api\n"
                    "api.lib().openfish_decode_cpu(1, 1, 256, 1, None, 3, None, None, None, None)\nprint('survived')")
    assert r.returncode != 0 and "survived" not in r.stdout
    assert "GPU path only" in r.stderr


def test_missing_library_fails_the_import(tmp_path):
    # the package must not fall back to anything when its shared library is absent
    pkg = tmp_path / "openfish_amd"
    pkg.mkdir()
    for f in ("__init__.py", "api.py"):
        (pkg / f).write_text(open(os.path.join(ROOT, "openfish_amd", f)).read())
    r = subprocess.run([sys.executable, "-c", "import sys; sys.path.insert(0, %r); import openfish_amd.api" % str(tmp_path)],
                       capture_output=True, text=True)
    assert r.returncode != 0 and "no CPU fallback" in r.stderr


def test_product_never_touches_the_oracle():
    for dirpath, _, files in os.walk(os.path.join(ROOT, "openfish_amd")):
        for f in files:
            if f.endswith((".py", ".c", ".h", ".hip")):
                text = open(os.path.join(dirpath, f)).read()
                assert "crf_oracle" not in text and "oracle/" not in text, os.path.join(dirpath, f)
    text = open(os.path.join(ROOT, "Makefile")).read()
    assert "libcrf_oracle" not in text
