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
    L.max_err_exp.restype = C.c_double
    L.max_err_exp.argtypes = [fp, C.c_long, C.c_int]
    L.max_abs_err_log_tab.restype = C.c_double
    L.max_abs_err_log_tab.argtypes = [fp, C.c_long]
    L.lse5_mismatches.restype = C.c_long
    L.lse5_mismatches.argtypes = [fp, C.c_long]
    L.max_abs_err_log_near.restype = C.c_double
    L.max_abs_err_log_near.argtypes = [fp, C.c_long, C.c_int]
    L.two_tier_wrongly_settled.restype = C.c_long
    L.two_tier_wrongly_settled.argtypes = [fp, C.c_long, C.POINTER(C.c_long), C.POINTER(C.c_long)]
    return L


def fptr(a):
    return a.ctypes.data_as(C.POINTER(C.c_float))


def test_exp_error_bounds(lib):
    """absolute error below 2^-51 everywhere (the sums these values enter are at least 1); relative
    error below 2^-50 where the value is not small and below 2^-48 down to e^-20, under which a
    term cannot change an fp32 sum that contains a 1"""
    rng = np.random.default_rng(1)
    near = np.concatenate([-5.5 * rng.random(400000), -1e-3 * rng.random(100000), -(np.arange(0, 176) / 32.0),
                           [0.0, -0.0, -1e-30]]).astype(np.float32)
    mid = np.concatenate([-20 * rng.random(400000), -(np.arange(0, 640) / 32.0)]).astype(np.float32)
    far = np.concatenate([-100 * rng.random(400000), -(np.arange(0, 3200) / 32.0), [-79.99999, -700.0]]).astype(np.float32)
    assert lib.max_err_exp(fptr(near), near.size, 1) < 2.0 ** -50
    assert lib.max_err_exp(fptr(mid), mid.size, 1) < 2.0 ** -48
    assert lib.max_err_exp(fptr(far), far.size, 0) < 2.0 ** -51


def test_exp_of_zero_is_exactly_one_and_far_tail_is_zero(lib):
    one = np.zeros(1, np.float32)
    assert lib.max_err_exp(fptr(one), 1, 1) == 0.0
    far = np.array([-20000.0, -1e8], np.float32)
    assert lib.max_err_exp(fptr(far), 2, 0) == 0.0  # exactly zero, like exp()


def test_table_log_absolute_error_below_2_pow_minus_51(lib):
    rng = np.random.default_rng(4)
    s = np.concatenate([1 + 4 * rng.random(500000), 1 + 1e-4 * rng.random(100000),
                        [1.0, 5.0, 2.0, 4.0, 1.015625, 1.9999999, 3.9999998,
                         np.nextafter(np.float32(1), np.float32(2))]]).astype(np.float32)
    assert lib.max_abs_err_log_tab(fptr(s), s.size) < 2.0 ** -51


def test_log_with_a_cell_chosen_from_a_neighbour(lib):
    """the second tier fetches the table cell with the fp32 estimate of the sum, which may lie a few
    ulps away from the sum itself, on the other side of a cell or binade boundary"""
    rng = np.random.default_rng(5)
    edges = 1 + np.arange(0, 129) / 32.0  # cell boundaries of [1, 5]
    s = np.concatenate([1 + 4 * rng.random(300000), edges, np.nextafter(edges.astype(np.float32), np.float32(9)),
                        np.nextafter(edges.astype(np.float32), np.float32(0)), [2.0, 4.0, 1.9999999, 3.9999998]]).astype(np.float32)
    s = s[(s >= 1) & (s <= 5)]
    assert lib.max_abs_err_log_near(fptr(s), s.size, 0) < 2.0 ** -51
    assert lib.max_abs_err_log_near(fptr(s), s.size, 40) < 2.0 ** -51  # 40 ulps: 5e-6 relative


@pytest.mark.parametrize("centre,spread", [(0.0, 3.0), (37.0, 2.0), (5900.0, 4.0), (5900.0, 40.0), (48000.0, 30.0),
                                           (-3000.0, 0.3), (700.0, 9.0)])
def test_lse5_reproduces_the_libm_roundings(lib, centre, spread):
    """the scan update with these routines vs. the same update with libm exp/log: the
    expected number of differing results is far below one in a million"""
    rng = np.random.default_rng(int(abs(centre)) + 7)
    v = (centre + spread * rng.standard_normal((1000000, 5))).astype(np.float32)
    assert lib.lse5_mismatches(fptr(v), v.shape[0]) == 0


@pytest.mark.parametrize("centre,spread,max_open", [(0.0, 3.0, 1.0), (100.0, 3.0, 0.25), (700.0, 3.0, 0.03),
                                                    (3000.0, 3.0, 0.008), (5900.0, 3.0, 0.004), (5900.0, 40.0, 0.002),
                                                    (48000.0, 30.0, 0.0003), (-3000.0, 0.3, 0.009), (-5000.0, 3.0, 0.004)])
def test_two_tier_estimate_is_never_wrongly_settled(lib, centre, spread, max_open):
    """the fp32 estimate of the scan update declares itself settled only where it equals the libm
    result; the fraction left to the double arithmetic shrinks as an ulp of the values grows.
    (Host build: libm's exp2f/log2f stand in for v_exp_f32/v_log_f32, whose measured error bounds
    are the larger ones and are what the bound in dmath.h budgets for.)"""
    rng = np.random.default_rng(int(abs(centre)) + 11)
    v = (centre + spread * rng.standard_normal((400000, 5))).astype(np.float32)
    unsettled, mismatches = C.c_long(), C.c_long()
    wrong = lib.two_tier_wrongly_settled(fptr(v), v.shape[0], C.byref(unsettled), C.byref(mismatches))
    assert wrong == 0 and mismatches.value == 0
    assert unsettled.value <= max_open * v.shape[0]


def test_two_tier_special_values_are_left_to_the_double_arithmetic(lib):
    """results that are zero or tiny never count as settled; a power of two may, and is then right"""
    cases = np.array([[0.0, -90.0, -90.0, -90.0, -90.0],      # exactly 0 + log(1 + tiny)
                      [1e-3, -1.0, -2.0, -3.0, -4.0],
                      [-2.5, -2.5, -2.5, -2.5, -2.5],
                      [4096.0, 3000.0, 3000.0, 3000.0, 3000.0]], np.float32)  # a power of two
    unsettled, mismatches = C.c_long(), C.c_long()
    wrong = lib.two_tier_wrongly_settled(fptr(cases[:3]), 3, C.byref(unsettled), C.byref(mismatches))
    assert wrong == 0 and mismatches.value == 0 and unsettled.value == 3
    wrong = lib.two_tier_wrongly_settled(fptr(cases), 4, C.byref(unsettled), C.byref(mismatches))
    assert wrong == 0 and mismatches.value == 0


@pytest.mark.parametrize("power", [4.0, 8.0, 64.0, 512.0, 4096.0, 32768.0, -8.0, -512.0])
def test_two_tier_results_next_to_a_power_of_two(lib, power):
    """the rounding boundary below a power of two is half as far away as the one above it: results
    scattered closely around +-2^k (the sum is 1 + one more term, chosen so that max + log(sum)
    lands within a few ulps of the power) must never be settled on the wrong side"""
    rng = np.random.default_rng(int(abs(power)) + 5)
    n = 300000
    gap = rng.uniform(1e-3 + 4.0 * np.spacing(np.float32(abs(power))), np.log(2.0), n)  # power - max
    big = power - gap
    ulps = rng.uniform(-3.0, 3.0, n) * np.spacing(np.float32(abs(power)))
    other = big + np.log(np.expm1(gap + ulps))          # exp(other - big) = exp(gap) - 1
    v = np.stack([big, other, big - 200.0, big - 300.0, big - 400.0], axis=1).astype(np.float32)
    unsettled, mismatches = C.c_long(), C.c_long()
    wrong = lib.two_tier_wrongly_settled(fptr(v), n, C.byref(unsettled), C.byref(mismatches))
    assert wrong == 0 and mismatches.value == 0
    if abs(power) >= 64.0:  # below that, half an ulp is within the error bound and nothing is ever settled
        assert unsettled.value < n  # some are settled: the case does exercise the settled branch


@pytest.mark.parametrize("terms,centre", [(2, 300.0), (2, 3000.0), (4, 900.0), (4, 5000.0), (3, 2500.0)])
def test_two_tier_sums_next_to_a_binade_of_the_sum(lib, terms, centre):
    """sums of exponentials scattered closely around 2 and 4, where the ulp of the CPU path's
    partial sums doubles: `terms` values within a few 1e-7 of the maximum (and, for three terms,
    one a factor of two further down, which lands on 2 + 1/2 + ... as well as on sums just below
    and above 2 and 4 through the scatter), the rest far below"""
    rng = np.random.default_rng(terms * 1000 + int(centre))
    n = 400000
    top = (centre + rng.uniform(-40.0, 40.0, n)).astype(np.float32)
    v = np.empty((n, 5), np.float64)
    for k in range(5):
        if k < terms:
            v[:, k] = top.astype(np.float64) - np.abs(rng.normal(0.0, 3e-4 * (k > 0), n))
        else:
            v[:, k] = top.astype(np.float64) - rng.uniform(14.0, 40.0, n)
    order = rng.permuted(np.tile(np.arange(5), (n, 1)), axis=1)   # the maximum in any position
    v = np.take_along_axis(v, order, axis=1).astype(np.float32)
    unsettled, mismatches = C.c_long(), C.c_long()
    wrong = lib.two_tier_wrongly_settled(fptr(v), n, C.byref(unsettled), C.byref(mismatches))
    assert wrong == 0 and mismatches.value == 0
    assert unsettled.value < n
