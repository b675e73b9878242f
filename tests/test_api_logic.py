"""Every op logic of the library against the oracle, and its analytic backward
against its own central-difference backward, on the host cores and on the GPU.

Follows the reference's gradient tests (tests/operation/unary/*_gradient.cu,
tests/operation/binary/*_gradient.cu, examples/mini-gaussian-splatting/tests/*.cu):
random inputs, fp64, error = min(abs, rel), tolerance 1e-5.
"""
import zlib

import numpy as np
import pytest

from tests import _native, _oracle_ops
from tests._metrics import abs_or_rel

NAMES = sorted(_native.LOGICS)


def _run(oracle, name, device, cases=20):
    rng = np.random.default_rng(zlib.crc32(("api" + name).encode()))
    _, _, _, n_out = _native.LOGICS[name]
    for _ in range(cases):
        ops, k = _oracle_ops.sample_inputs(name, rng)
        up = rng.uniform(-1.5, 1.5, n_out)
        want_y, want_g = _oracle_ops.evaluate(oracle, name, ops, k, up, np.float64)
        y, analytic, numeric = _native.eval_logic(name, ops, k, up, np.float64, 1e-6, device)
        assert abs_or_rel(y, want_y).max() < 1e-12, (name, y, want_y)
        assert abs_or_rel(analytic, want_g).max() < 1e-11, (name, analytic, want_g)
        assert abs_or_rel(analytic, numeric).max() < 1e-5, (name, analytic, numeric)
        # fp32 build of the same templates against the fp32 oracle
        y32, a32, _ = _native.eval_logic(name, ops, k, up, np.float32, 1e-3, device)
        ops32 = [np.asarray(o, np.float32) for o in ops]
        w_y32, w_g32 = _oracle_ops.evaluate(oracle, name, ops32, np.asarray(k, np.float32), up.astype(np.float32), np.float32)
        assert abs_or_rel(y32, w_y32).max() < 2e-5, (name, y32, w_y32)
        assert abs_or_rel(a32, w_g32).max() < 2e-4, (name, a32, w_g32)


@pytest.mark.parametrize("name", NAMES)
def test_logic_on_host(oracle, name):
    _run(oracle, name, device=False)


@pytest.mark.gpu
@pytest.mark.parametrize("name", NAMES)
def test_logic_on_gpu(gpu, oracle, name):
    _run(oracle, name, device=True, cases=6)


def test_fp32_exp_and_sincos_are_accurate_to_two_ulp():
    """math::exp and math::sincos for float are the library's own implementations."""
    import ctypes

    lib = _native.load()
    xs = np.concatenate([np.linspace(-87, 88, 4001), np.linspace(-1e-3, 1e-3, 101)])
    out = np.zeros(64)
    worst = 0.0
    for x in xs[::7]:
        y, _, _ = _native.eval_logic("exp", [np.array([x, x / 2, -x])], dtype=np.float32)
        ref = np.exp(np.float64(np.float32(np.array([x, x / 2, -x]))))
        ulp = np.spacing(ref.astype(np.float32)).astype(np.float64)
        worst = max(worst, (np.abs(y - ref) / ulp).max())
    assert worst <= 2.0, worst
    worst = 0.0
    for x in np.concatenate([np.linspace(-3.2, 3.2, 801), np.linspace(-100, 100, 401), [1000.5, -4097.25, 8000.0, 9000.0, 1e6]]):
        s, _, _ = _native.eval_logic("sin", [np.array([x, -x, x / 3])], dtype=np.float32)
        c, _, _ = _native.eval_logic("cos", [np.array([x, -x, x / 3])], dtype=np.float32)
        arg = np.float64(np.float32(np.array([x, -x, x / 3])))
        worst = max(worst, np.abs(s - np.sin(arg)).max(), np.abs(c - np.cos(arg)).max())
    assert worst <= 2.5e-7, worst  # absolute: two ulp of values near one


def _special_values(device):
    inf, big = np.inf, float(np.finfo(np.float32).max)
    e, _, _ = _native.eval_logic("exp", [np.array([-inf, -big, -104.0])], dtype=np.float32, device=device)
    assert np.all(e == 0.0), e
    e, _, _ = _native.eval_logic("exp", [np.array([inf, big, 89.0])], dtype=np.float32, device=device)
    assert np.all(e == inf), e
    e, _, _ = _native.eval_logic("exp", [np.array([np.nan, 0.0, -0.0])], dtype=np.float32, device=device)
    assert np.isnan(e[0]) and e[1] == 1.0 and e[2] == 1.0, e
    s, _, _ = _native.eval_logic("sigmoid", [np.array([inf, big, 200.0])], dtype=np.float32, device=device)
    assert np.all(s == 1.0), s
    s, _, _ = _native.eval_logic("sigmoid", [np.array([-inf, -big, -200.0])], dtype=np.float32, device=device)
    assert np.all(s == 0.0), s


def test_fp32_exp_and_sigmoid_at_the_ends_of_the_range():
    """expf of the C library gives 0 at -inf and below the range, inf above it; sigmoid follows with 0 and 1."""
    _special_values(device=False)


@pytest.mark.gpu
def test_fp32_exp_and_sigmoid_at_the_ends_of_the_range_on_gpu(gpu):
    _special_values(device=True)
