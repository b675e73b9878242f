"""The library's gradient testers (xyz_autodiff/testing/unary_gradient_tester.cuh,
binary_gradient_tester.cuh, network_gradient_tester.cuh) used exactly as the tests of
xyz-autodiff-cuda use theirs: all 94 Unary/BinaryGradientTester calls (tests/operation/unary/*_gradient.cu,
tests/operation/binary/*_gradient.cu, tests/operation/base/test_gradient_verification.cu,
tests/operation/unary/test_norm_operations.cu, test_sym_matrix2_inv.cu,
examples/mini-gaussian-splatting/tests/*.cu) and the 6 NetworkGradientTester calls
(tests/operation/base/test_linear_regression_network.cu:199-317), with their logic types, dimensions,
case counts, tolerances (1e-5; 1e-3 for the large-value network), deltas and input ranges.
"""
import pytest

from tests import _native

CALLS = 100
SELF_CHECKS = (1 << 10) - 1


def _check(rows, bits, device):
    assert len(rows) == CALLS
    failing = [r for r in rows if r[3] != 0]
    assert not failing, failing
    assert all(r[5] == device for r in rows), "cases ran on the wrong side"
    assert all(r[2] > 0 for r in rows)
    # the tolerance every call passes is the one its reference test names; the errors are far below it
    assert max(r[4] for r in rows if "LargeValues" not in r[1]) < 1e-5
    # a wrong sign, a forgotten operand gradient and an inconsistent network are reported;
    # a loosened or negative tolerance is refused; see run_self_checks() in tests/native/tester_suite.cuh
    assert bits == SELF_CHECKS, bin(bits)
    files = {r[0].rsplit(":", 1)[0] for r in rows}
    assert len(files) == 17, sorted(files)


def test_reference_tester_calls_on_host():
    rows, bits = _native.run_tester_suite(device=False)
    _check(rows, bits, device=False)


@pytest.mark.gpu
def test_reference_tester_calls_on_gpu(gpu):
    rows, bits = _native.run_tester_suite(device=True)
    _check(rows, bits, device=True)
