"""GPU parity of the least-squares example (fp64, four shared parameters), through the C ABI.

Truth: the oracle's fp64 sums.  The GPU adds the same fp64 terms in another
order, so a sum may differ by the rounding of the summation: a few ulp of the
mass of the terms, sum |g_i|.  The bound used is 1e-12 of that mass for the
staged strategies (thousands of partial sums) and for the naive one.
"""
import numpy as np
import pytest

from xyz_autodiff_cuda_amd import linreg

pytestmark = pytest.mark.gpu

STRATEGIES = ["global_atomics", "lds_leaves", "wave_lds"]


def _mass(p, x1, x2, y):
    a, b, c, d = p
    r = (x1 - a) ** 2 + b * (x2 - c) ** 2 + d - y
    g = np.stack([4.0 * r * (x1 - a), 2.0 * r * (x2 - c) ** 2, 4.0 * r * b * (x2 - c), 2.0 * r, r * r])
    return np.abs(g).sum(axis=1)


def _device(gpu, *arrays):
    import torch

    return [torch.from_numpy(np.ascontiguousarray(a)).to(gpu) for a in arrays]


@pytest.mark.parametrize("strategy", STRATEGIES)
@pytest.mark.parametrize("n", [1, 63, 64, 255, 257, 8192, 100_000, 1_000_003])
def test_gradient_matches_oracle(gpu, oracle, strategy, n):
    import torch

    x1, x2, y = linreg.synthetic_data(n, seed=n)
    p = np.array([0.4, 1.3, -0.2, 0.1])
    want = oracle.linreg_gradient(x1, x2, y, p)
    dx1, dx2, dy, dp = _device(gpu, x1, x2, y, p)
    out = torch.full((5,), 123.0, dtype=torch.float64, device=gpu)  # overwritten, not added to
    got = linreg.batch_gradient(dx1, dx2, dy, dp, strategy=strategy, out=out).cpu().numpy()
    assert np.all(np.abs(got - want) <= 1e-12 * _mass(p, x1, x2, y) + 1e-300), (got, want)


@pytest.mark.parametrize("strategy", STRATEGIES)
def test_gradient_with_rows(gpu, oracle, strategy):
    total, n = 100_000, 8192  # the reference's data set and batch (linear_regression_sgd.cu:23-24)
    x1, x2, y = linreg.synthetic_data(total, seed=1)
    rows = np.random.default_rng(3).integers(0, total, n).astype(np.int32)
    p = np.array(linreg.INITIAL_PARAMS)
    want = oracle.linreg_gradient(x1, x2, y, p, rows)
    dx1, dx2, dy, dp, drows = _device(gpu, x1, x2, y, p, rows)
    got = linreg.batch_gradient(dx1, dx2, dy, dp, rows=drows, strategy=strategy).cpu().numpy()
    assert np.all(np.abs(got - want) <= 1e-12 * _mass(p, x1[rows], x2[rows], y[rows]))


@pytest.mark.parametrize("strategy", STRATEGIES)
def test_reference_points(gpu, oracle, strategy):
    # the five single-sample cases and the 32-sample batch of test_linear_regression_gradient.cu:160-233
    from tests.test_oracle_linreg import REFERENCE_POINTS

    for point, params in REFERENCE_POINTS:
        x1, x2, y = (np.array([v]) for v in point)
        want = oracle.linreg_gradient(x1, x2, y, params)
        got = linreg.batch_gradient(*_device(gpu, x1, x2, y, np.array(params)), strategy=strategy).cpu().numpy()
        np.testing.assert_allclose(got, want, rtol=1e-14, atol=1e-300)
    i = np.arange(32, dtype=np.float64)
    x1, x2, y, p = i * 0.1, i * 0.2, i * 0.3 + 1.0, np.array([0.5, 1.0, 0.3, 0.1])
    got = linreg.batch_gradient(*_device(gpu, x1, x2, y, p), strategy=strategy).cpu().numpy()
    np.testing.assert_allclose(got, oracle.linreg_gradient(x1, x2, y, p), rtol=1e-13)


def test_empty_batch_and_out_of_range_rows(gpu, oracle):
    import torch

    x1, x2, y = linreg.synthetic_data(100, seed=9)
    p = np.array(linreg.TRUE_PARAMS)
    dx1, dx2, dy, dp = _device(gpu, x1, x2, y, p)
    empty = torch.empty(0, dtype=torch.int32, device=gpu)
    assert torch.all(linreg.batch_gradient(dx1, dx2, dy, dp, rows=empty) == 0)
    rows = np.array([5, -1, 100, 7, 2_000_000_000, 5], dtype=np.int32)  # three valid rows; the rest is dropped
    want = oracle.linreg_gradient(x1, x2, y, p, np.array([5, 7, 5], dtype=np.int32))
    for strategy in STRATEGIES:
        got = linreg.batch_gradient(dx1, dx2, dy, dp, rows=_device(gpu, rows)[0], strategy=strategy).cpu().numpy()
        np.testing.assert_allclose(got, want, rtol=1e-13)


def test_bad_arguments(gpu, xad):
    import torch

    x = torch.zeros(4, dtype=torch.float64, device=gpu)
    with pytest.raises(xad.XadError):
        linreg.batch_gradient(x, x, x, x, strategy=9)
    with pytest.raises(ValueError):
        linreg.batch_gradient(x.float(), x, x, x)
    with pytest.raises(xad.XadError):
        linreg.sgd(x, x, x, x.clone(), batch=0, epochs=1)


def test_device_draw_matches_host_draw(gpu, oracle):
    # one SGD step with a learning rate so small that params stay put: the loss history is the mean
    # loss over the rows the device drew, which must be the rows the host restatement lists
    import torch

    total, batch = 100_000, 8192
    x1, x2, y = linreg.synthetic_data(total, seed=4)
    dx1, dx2, dy = _device(gpu, x1, x2, y)
    params = torch.tensor(linreg.INITIAL_PARAMS, dtype=torch.float64, device=gpu)
    hist = linreg.sgd(dx1, dx2, dy, params, batch, 3, lr_first=1e-300, lr_last=1e-300, seed=17, want_history=True).cpu().numpy()
    for e in range(3):
        rows = linreg.batch_rows(17, e, batch, total)
        assert rows.min() >= 0 and rows.max() < total and len(np.unique(rows)) > batch * 0.9
        want = oracle.linreg_gradient(x1, x2, y, linreg.INITIAL_PARAMS, rows)[4] / batch
        np.testing.assert_allclose(hist[e], want, rtol=1e-12)


# the reference batch, a batch smaller than one launch grid, and one of most of the data set
@pytest.mark.parametrize("batch,epochs", [(8192, 300), (1000, 50), (70_000, 40)])
def test_sgd_trajectory_matches_oracle(gpu, oracle, batch, epochs):
    import torch

    total = 100_000
    x1, x2, y = linreg.synthetic_data(total, seed=6)
    rows = np.concatenate([linreg.batch_rows(5, e, batch, total) for e in range(epochs)])
    want_p, want_hist = oracle.linreg_sgd(x1, x2, y, rows, linreg.INITIAL_PARAMS, batch, epochs, 1e-4, 1e-6)
    params = torch.tensor(linreg.INITIAL_PARAMS, dtype=torch.float64, device=gpu)
    hist = linreg.sgd(*_device(gpu, x1, x2, y), params, batch, epochs, 1e-4, 1e-6, seed=5, want_history=True).cpu().numpy()
    # summation order differs per step (1e-16 relative); the iteration contracts, so the difference stays small
    np.testing.assert_allclose(params.cpu().numpy(), want_p, rtol=1e-9, atol=1e-10)
    np.testing.assert_allclose(hist, want_hist, rtol=1e-9)
    assert hist[-1] < (0.5 if epochs >= 300 else 1.0) * hist[0]


def test_sgd_reference_hyperparameters_converge(gpu):
    # linear_regression_sgd.cu:23-28: 100 000 samples, batch 8192, 10 000 steps, lr 1e-4 -> 1e-6, noise 0.5
    import torch

    x1, x2, y = linreg.synthetic_data(100_000, seed=0, noise=0.5)
    params = torch.tensor(linreg.INITIAL_PARAMS, dtype=torch.float64, device=gpu)
    hist = linreg.sgd(*_device(gpu, x1, x2, y), params, 8192, 10_000, seed=1, want_history=True).cpu().numpy()
    p = params.cpu().numpy()
    assert np.all(np.isfinite(p)) and np.all(np.isfinite(hist))
    np.testing.assert_allclose(p[:3], linreg.TRUE_PARAMS[:3], atol=0.05)
    assert hist[-1] < 2e-3 * hist[0]
