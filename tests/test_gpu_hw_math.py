"""The premises of the two-tier arithmetic, measured on the device the tests run on.

The default scan mode (openfish_amd/csrc/dmath.h, lse5_estimate) and the beam search's merges
(openfish_amd/csrc/beam.hip, log_sum_exp_estimate) take the hardware's fp32 exp2/log2 where a
bound on everything that separates the estimate from the CPU path's value (reference
src/decode_cpu.c:45-49, src/beam_search.c:43-47) proves that both round to the same fp32 number.
Those bounds budget the hardware's own errors: 1.43 units of 2^-24 (relative) for v_exp_f32 on
[-160, 0], and 1.0 / 2.0 / 4.0 units (absolute) for v_log_f32 on [1,2) / [2,4) / [4,5.01], and
they use exp2(0) = 1 and log2(1) = 0.  A device or compiler whose instructions are worse than that
would make the default mode differ from the CPU path without any other test necessarily noticing;
this test sweeps every fp32 input of those ranges (1.1e9 + 1.9e7 values) against double arithmetic.
"""
import pytest

pytestmark = pytest.mark.gpu



@pytest.fixture(scope="module")
def api():
    from openfish_amd import api as _api
    if _api.device_count() < 1:
        pytest.skip("no HIP device")
    return _api


# what the derivations in dmath.h (lse5_estimate) and beam.hip (log_sum_exp_estimate) budget
EXP_REL_BUDGET = 1.43
LOG_ABS_BUDGET = (1.0, 2.0, 4.0)


def test_hardware_exp2_and_log2_stay_within_the_budgeted_errors(api):
    errors, identities = api.probe_hw_math()
    print("v_exp_f32 rel %.4f, v_log_f32 abs %.4f %.4f %.4f (units of 2^-24), identities %s"
          % (errors[0], errors[1], errors[2], errors[3], bin(identities)))
    assert 0.5 < errors[0] <= EXP_REL_BUDGET, errors  # far below: the sweep did not run
    for got, budget in zip(errors[1:], LOG_ABS_BUDGET):
        assert 0.25 * budget < got <= budget, errors
    assert identities & 1, "exp2(0) != 1"
    assert identities & 2, "exp2(-0) != 1"
    assert identities & 4, "log2(1) != 0"
    assert identities & 8, "log2(2) != 1"
