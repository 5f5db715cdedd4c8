"""Accuracy of the double-precision exp/log written for the scans
(openfish_amd/csrc/dmath.h), host build, against long-double libm."""
import ctypes as C
import os
import subprocess

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib(tmp_path_factory):
    so = str(tmp_path_factory.mktemp("dmath") / "dmath_host.so")
    subprocess.check_call(["g++", "-O2", "-shared", "-fPIC", "-ffp-contract=off",
                           "-I", os.path.join(ROOT, "openfish_amd", "csrc"),
                           os.path.join(ROOT, "tests", "dmath_host.cpp"), "-o", so, "-lm"])
    L = C.CDLL(so)
    fp = C.POINTER(C.c_float)
    L.max_rel_err_exp.restype = C.c_double
    L.max_rel_err_exp.argtypes = [fp, C.c_long]
    L.max_rel_err_log.restype = C.c_double
    L.max_rel_err_log.argtypes = [fp, C.c_long]
    L.max_abs_err_lse2.restype = C.c_double
    L.max_abs_err_lse2.argtypes = [fp, C.c_long]
    L.lse2_mismatches.restype = C.c_long
    L.lse2_mismatches.argtypes = [fp, C.c_long]
    L.max_rel_err_exp_ldexp.restype = C.c_double
    L.max_rel_err_exp_ldexp.argtypes = [fp, C.c_long]
    L.max_abs_err_log_tab.restype = C.c_double
    L.max_abs_err_log_tab.argtypes = [fp, C.c_long]
    L.lse5_mismatches.restype = C.c_long
    L.lse5_mismatches.argtypes = [fp, C.c_long]
    return L


def fptr(a):
    return a.ctypes.data_as(C.POINTER(C.c_float))


def test_exp_relative_error_below_2_pow_minus_46(lib):
    rng = np.random.default_rng(1)
    d = np.concatenate([-80 * rng.random(400000), -rng.random(200000), -1e-3 * rng.random(100000),
                        -(np.arange(0, 2560) / 32.0), [0.0, -0.0, -1e-30, -79.99999]]).astype(np.float32)
    assert lib.max_rel_err_exp(fptr(d), d.size) < 2.0 ** -50


def test_ldexp_scaled_exp_and_table_log(lib):
    rng = np.random.default_rng(4)
    d = np.concatenate([-100 * rng.random(400000), -rng.random(100000), [0.0, -700.0]]).astype(np.float32)
    assert lib.max_rel_err_exp_ldexp(fptr(d), d.size) < 2.0 ** -50
    far = np.array([-745.0, -20000.0, -1e8], np.float32)  # subnormal or zero results: absolute check
    assert lib.max_rel_err_exp_ldexp(fptr(far[1:]), 2) == 0.0  # exactly zero, like exp()
    s = np.concatenate([1 + 4 * rng.random(500000), 1 + 1e-4 * rng.random(100000),
                        [1.0, 5.0, 2.0, 4.0, 1.015625, 1.9999999, 3.9999998]]).astype(np.float32)
    assert lib.max_abs_err_log_tab(fptr(s), s.size) < 2.0 ** -51


def test_exp_of_zero_is_exactly_one_and_far_tail_is_tiny(lib):
    one = np.zeros(1, np.float32)
    assert lib.max_rel_err_exp(fptr(one), 1) == 0.0


def test_log_relative_error_below_2_pow_minus_51(lib):
    rng = np.random.default_rng(2)
    s = np.concatenate([1 + 4 * rng.random(500000), 1 + 1e-3 * rng.random(100000), 1 + 1e-6 * rng.random(50000),
                        [1.0, 5.0, 2.0, 4.0, np.sqrt(2), 2 * np.sqrt(2), 1.4142135, 1.4142137,
                         np.nextafter(np.float32(1), np.float32(2))]]).astype(np.float32)
    assert lib.max_rel_err_log(fptr(s), s.size) < 2.0 ** -51


@pytest.mark.parametrize("centre,spread", [(0.0, 3.0), (37.0, 2.0), (5900.0, 4.0), (5900.0, 40.0), (48000.0, 30.0)])
def test_lse5_reproduces_the_libm_roundings(lib, centre, spread):
    """the scan update with these routines vs. the same update with libm exp/log: the
    expected number of differing results is far below one in a million"""
    rng = np.random.default_rng(int(centre) + 7)
    v = (centre + spread * rng.standard_normal((1000000, 5))).astype(np.float32)
    assert lib.lse5_mismatches(fptr(v), v.shape[0]) == 0


def test_pairwise_log_sum_exp_correction(lib):
    rng = np.random.default_rng(3)
    gap = np.concatenate([17 * rng.random(500000), 1e-3 * rng.random(50000), [0.0, 16.999998, 1e-30]]).astype(np.float32)
    assert lib.max_abs_err_lse2(fptr(gap), gap.size) < 2.0 ** -46
    for centre in (0.0, 40.0, 6000.0):
        xy = (centre + 5 * rng.standard_normal((1000000, 2))).astype(np.float32)
        assert lib.lse2_mismatches(fptr(xy), xy.shape[0]) == 0
