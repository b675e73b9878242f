"""Known answers for the public operator API, on the host cores and on the GPU.

The cases are in tests/native/api_cases.cuh, each a restatement of a test of the
reference (file and lines cited there); the numbers below are the ones those
tests expect.  The same compiled case functions run on both sides.
"""
import math

import numpy as np
import pytest

from tests import _native

E = math.e

EXPECTED = {
    0: [1, 2, 3, 0, 2, 4, 0, 0, 0],
    1: [10, 11, 12, 0, 3, 6, 3.5, 7.5, 7.5, 1.25, -2.5, 0],
    2: [1, 2, 3, 4, 5, 6, 1, 4, 2, 5, 3, 6, 2.5, 0],
    3: [19, 22, 43, 50, 17, 23, 39, 53],
    4: [1, 0, 0, 0, 2, 0, 0, 0, 3] + [1, 2, 6, 8, 15, 18] + [1, 4, 9, 4, 10, 18] + [2, 4, 0, 3],
    5: [1, 2, 2, 4, 3, 6, 2, 5] + [1, 2, 2, 4, 5, 5] + [1, 2, 3, 4, 5, 6] + [6, 10] + [1, 2, 3],
    6: [5, 7, 9, 3, 3, 3, 4, 10, 18, 4, 2.5, 2] + [4, 6, 8] + [4, 4, 4] + [2, 3, 4] + [-2, -3, -4] + [14, 18],
    7: [3.5, 4.5, 5.5, 1, 1, 1] + [0.5, 1.5, 2.5, 1, 1, 1] + [1.5, 3, 4.5, 1.5, 1.5, 1.5] + [1 / 3, 2 / 3, 1, 1 / 3, 1 / 3, 1 / 3],
    8: [6, -2.5, 1, 1] + [-2, -3.5, 1, -1] + [8, -1.5, 4, 0.5, 2, -3] + [0.5, -6, 0.25, 2, -0.125, 12],
    9: [3.5] * 4 + [10] + [3, 5, 7] + [3] + [1, 1, 1] + [1.5, 6],
    10: [6, 4] + [9, 4] + [12, 7] + [-1.2, 2, 2] + [12, 8, 6, 16],
    11: [2.5, 1.5, 0.75, 1.125, 1.5, 0.75, 1.125],
    12: [4.625, 2.5, -3.5] + [2 * (E + E ** -2), 2 * E, 2 * E ** -2],
    # TernaryOperation, y = a b + c: values; d a = b, d b = a, d c = 1 (analytic, then numerical);
    # node operands: e^0.6 - 0.3, 2 e^0.6 - 1; a ternary node consumed twice: 3.5 + 3.5^2, 8 (b, a, 1)
    16: [1.0, -7.0] + [0.5, 3.0, 1.5, -2.0, 1.0, 1.0] * 2 + [E ** 0.6 - 0.3, 2 * E ** 0.6 - 1] + [15.75, 12.0, 16.0, 8.0],
    # roots sharing a node: 0 until the last root has released it, then (2 s - 1) s with s = e^0.5
    17: [0.0, -E ** 0.5, E, (2 * E ** 0.5 - 1) * E ** 0.5] + [E ** 0.5, 2 * E ** 0.5] + [0.0, (2 * E ** 0.5 - 1) * E ** 0.5]
        + [3 * (E ** 0.5 + E), 3 * (E ** 0.25 + E ** 0.5), 3 * (E ** 0.25 + 2 * E ** 0.5)],
}


def _math_expectations():
    x = 1.0
    sig = lambda v: 1 / (1 + math.exp(-v))
    gelu = 0.5 * x * (1 + math.tanh(0.7978845608028654 * (x + 0.044715 * x ** 3)))
    return [math.exp(x), 1.0, math.sin(x), math.cos(x), math.tan(x), math.sinh(x), math.cosh(x), math.tanh(x), 2.0, 8.0,
            2.5, 2.0, 1.0, 0.5, 0.0, 2.0, -0.01, math.exp(-1) - 1, math.log(2), sig(1.0), gelu, math.sin(2.5), math.cos(2.5)]


def _regression_network_expectations():
    """Closed form of loss = ((a - x1)^2 + b (c - x2)^2 + d - y)^2 at the four parameter sets of
    tests/operation/base/test_linear_regression_network.cu; per set: loss, 4 analytic, 4 numerical gradients."""
    sets = [(1.0, 1.5, 0.5, 0.2, 2.0, 1.5, 3.0), (0.8, 1.2, -0.3, 0.5, 1.0, 0.8, 2.5),
            (10.0, 15.0, -8.0, 5.0, 20.0, -10.0, 100.0), (0.001, 0.002, -0.001, 0.0001, 0.01, -0.01, 0.001)]
    out = []
    for a, b, c, d, x1, x2, y in sets:
        r = (a - x1) ** 2 + b * (c - x2) ** 2 + d - y
        g = [4 * r * (a - x1), 2 * r * (c - x2) ** 2, 4 * r * b * (c - x2), 2 * r]
        out.append([r * r] + g + g)
    return out


def _check(case_id, got):
    if case_id == 15:
        # analytic gradients to rounding; numerical ones to the reference's tolerances for these sets
        # (1e-5, 1e-5, 1e-3 for the large values, 1e-5), measured like its testers: min(abs, rel)
        assert len(got) == 4 * 9
        for k, (want, tol) in enumerate(zip(_regression_network_expectations(), (1e-5, 1e-5, 1e-3, 1e-5))):
            block = np.asarray(got[9 * k:9 * k + 9])
            want = np.asarray(want)
            assert np.allclose(block[:5], want[:5], rtol=1e-12, atol=1e-300), (k, block, want)
            err = np.abs(block[5:] - want[5:])
            assert np.all(np.minimum(err, err / (np.abs(want[5:]) + 1e-300)) <= tol), (k, block, want)
        return
    if case_id in (13, 14):
        want = _math_expectations()
        tol = 1e-6 if case_id == 13 else 1e-12  # fp32: tests/test_math_dispatcher.cu uses 1e-5; fp64: 1e-10
    else:
        want = EXPECTED[case_id]
        tol = 1e-6
    assert len(got) == len(want), (case_id, len(got), len(want))
    assert np.allclose(got, want, rtol=tol, atol=tol), (case_id, list(got), want)


@pytest.mark.parametrize("case_id", sorted(EXPECTED) + [13, 14, 15])
def test_case_on_host(case_id):
    _check(case_id, _native.run_case(case_id, device=False))


@pytest.mark.gpu
@pytest.mark.parametrize("case_id", sorted(EXPECTED) + [13, 14, 15])
def test_case_on_gpu(gpu, case_id):
    got = _native.run_case(case_id, device=True)
    _check(case_id, got)
    host = _native.run_case(case_id, device=False)
    # 15 holds finite differences, which amplify the last-bit differences between the two builds
    tol = {13: 2e-6, 15: 1e-5}.get(case_id, 1e-12)
    assert np.allclose(got, host, rtol=tol, atol=tol)


@pytest.mark.gpu
@pytest.mark.parametrize("threads,block", [(10_000, 256), (100_000, 512)])
def test_concurrent_add_grad_on_global_memory(gpu, threads, block):
    """tests/test_parallel_gradient_accumulation.cu:94-110 and :162-167 of the reference."""
    got = _native.parallel_accumulation(threads, block)
    assert got[0] == threads and got[1] == threads
    want = 3.0 * threads + 0.002 * (threads - 1) * threads / 2
    assert abs(got[2] - want) <= 1e-6 * want


@pytest.mark.gpu
@pytest.mark.parametrize("blocks,threads", [(1, 128), (4, 64)])
def test_concurrent_add_grad_on_lds(gpu, blocks, threads):
    """tests/test_shared_memory_atomic.cu:102-109 and :179-187 of the reference."""
    got = _native.shared_accumulation(blocks, threads)
    assert np.all(got[:, 0] == threads) and np.all(got[:, 1] == 2 * threads)


@pytest.mark.gpu
@pytest.mark.parametrize("threads", [1, 64, 10_000, 1 << 20])
def test_concurrent_add_grad_on_managed_memory(gpu, threads):
    """VariableRef over makeHipManagedArray memory, the pairing of the reference's tests (cuda_managed_ptr,
    tests/test_parallel_gradient_accumulation.cu:60-99): no contribution may be lost, in float or double."""
    got = _native.managed_accumulation(threads)
    assert list(got) == [threads, 2.0 * threads, threads, 2.0 * threads], got
