"""Pins the least-squares oracle (oracle/oracle_linreg.c) and checks the library's
templates, compiled for the host, against it.  No GPU.

The reference holds no expected numbers for this graph: its tests compare the
analytic gradient with its own central differences
(examples/optimization/tests/test_linear_regression_gradient.cu:96-150).  The
pins here are therefore values worked out by hand for the reference's test
points, a closed form written independently of the graph, central differences
of an independently written loss, and properties of the SGD loop.
"""
import numpy as np
import pytest

from xyz_autodiff_cuda_amd import linreg

# (x1, x2, y), (a, b, c, d) of test_linear_regression_gradient.cu:160-215
REFERENCE_POINTS = [
    ((2.0, 3.0, 5.0), (1.0, 1.5, 0.5, 0.2)),
    ((1.0, 1.0, 2.0), (0.0, 0.0, 0.0, 0.0)),
    ((-2.0, -1.5, 3.0), (-1.0, 2.0, -0.5, -0.3)),
    ((100.0, 150.0, 500.0), (50.0, 30.0, 70.0, 20.0)),
    ((0.001, 0.002, 0.001), (0.0001, 0.0002, 0.0001, 0.00001)),
]


def loss_np(p, x1, x2, y):
    a, b, c, d = p
    return ((x1 - a) ** 2 + b * (x2 - c) ** 2 + d - y) ** 2


def closed_form(p, x1, x2, y):
    a, b, c, d = p
    r = (x1 - a) ** 2 + b * (x2 - c) ** 2 + d - y
    g = np.stack([-4.0 * r * (x1 - a), 2.0 * r * (x2 - c) ** 2, -4.0 * r * b * (x2 - c), 2.0 * r])
    return np.concatenate([g.sum(axis=1), [np.sum(r * r)]])


def test_hand_computed_points(oracle):
    # x = (2, 3), y = 5, p = (1, 1.5, 0.5, 0.2): (a-x1)^2 = 1, (c-x2)^2 = 6.25, prediction = 10.575, residual = 5.575
    out = oracle.linreg_gradient([2.0], [3.0], [5.0], REFERENCE_POINTS[0][1])
    np.testing.assert_allclose(out, [-22.3, 69.6875, -83.625, 11.15, 31.080625], rtol=1e-14)
    # x = (1, 1), y = 2, p = 0: prediction = 1, residual = -1
    out = oracle.linreg_gradient([1.0], [1.0], [2.0], REFERENCE_POINTS[1][1])
    np.testing.assert_allclose(out, [4.0, -2.0, 0.0, -2.0, 1.0], rtol=0, atol=0)


@pytest.mark.parametrize("point,params", REFERENCE_POINTS)
def test_reference_points_closed_form_and_differences(oracle, point, params):
    x1, x2, y = (np.array([v]) for v in point)
    out = oracle.linreg_gradient(x1, x2, y, params)
    np.testing.assert_allclose(out, closed_form(params, x1, x2, y), rtol=1e-13, atol=1e-300)
    p = np.array(params)
    scale = max(1.0, np.abs(out[:4]).max())
    for k in range(4):
        h = 1e-6 * max(1.0, abs(p[k]))
        hi, lo = p.copy(), p.copy()
        hi[k] += h
        lo[k] -= h
        fd = (loss_np(hi, x1, x2, y)[0] - loss_np(lo, x1, x2, y)[0]) / (2 * h)
        assert abs(fd - out[k]) <= 1e-7 * scale, (k, fd, out[k])


def test_batch_of_the_reference_test(oracle):
    # test_linear_regression_gradient.cu:219-233: 32 samples (0.1 i, 0.2 i, 0.3 i + 1), p = (0.5, 1, 0.3, 0.1)
    i = np.arange(32, dtype=np.float64)
    x1, x2, y = i * 0.1, i * 0.2, i * 0.3 + 1.0
    p = (0.5, 1.0, 0.3, 0.1)
    out = oracle.linreg_gradient(x1, x2, y, p)
    np.testing.assert_allclose(out, closed_form(p, x1, x2, y), rtol=1e-13)
    assert np.all(out != 0)


def test_rows_select_and_repeat_samples(oracle):
    rng = np.random.default_rng(5)
    x1, x2, y = rng.uniform(-5, 5, (3, 100))
    rows = rng.integers(0, 100, 1000).astype(np.int32)
    p = (0.3, 1.2, -0.4, 0.9)
    np.testing.assert_allclose(oracle.linreg_gradient(x1, x2, y, p, rows), closed_form(p, x1[rows], x2[rows], y[rows]), rtol=1e-12)


def test_host_templates_match_oracle(oracle, xad):
    rng = np.random.default_rng(11)
    x1, x2, y = rng.uniform(-5, 5, (3, 5000))
    rows = rng.integers(0, 5000, 3000).astype(np.int32)
    for p in [linreg.INITIAL_PARAMS, linreg.TRUE_PARAMS, (-3.0, 0.25, 4.0, -10.0)]:
        for r in (None, rows):
            want = oracle.linreg_gradient(x1, x2, y, p, r)
            got = linreg.host_batch_gradient(x1, x2, y, p, r)
            # same statements in the same order: only the compiler's contraction may differ
            np.testing.assert_allclose(got, want, rtol=1e-13)
    for point, params in REFERENCE_POINTS:
        got = linreg.host_batch_gradient([point[0]], [point[1]], [point[2]], params)
        np.testing.assert_allclose(got, oracle.linreg_gradient([point[0]], [point[1]], [point[2]], params), rtol=1e-14, atol=1e-300)


def test_host_rejects_bad_rows(xad):
    with pytest.raises(xad.XadError):
        linreg.host_batch_gradient([0.0], [0.0], [0.0], (0, 0, 0, 0), rows=[3])
    assert np.all(linreg.host_batch_gradient(np.zeros(0), np.zeros(0), np.zeros(0), (1, 2, 3, 4)) == 0)


def test_sgd_single_step_closed_form(oracle):
    rng = np.random.default_rng(2)
    x1, x2, y = rng.uniform(-5, 5, (3, 64))
    rows = np.arange(64, dtype=np.int32)
    p0 = np.array(linreg.INITIAL_PARAMS)
    p1, hist = oracle.linreg_sgd(x1, x2, y, rows, p0, 64, 1, 1e-4, 1e-6)
    sums = closed_form(p0, x1, x2, y)
    np.testing.assert_allclose(p1, p0 - 1e-4 * sums[:4] / 64, rtol=1e-13)  # lr(0) = lr_first
    np.testing.assert_allclose(hist[0], sums[4] / 64, rtol=1e-13)


def test_sgd_learning_rate_schedule(oracle):
    # One sample at x = 0 with a = b = c = 0: the residual is d - y and each step multiplies it by
    # 1 - 2 lr(e).  Read lr(e) back from the loss history and compare with
    # lr_first * (lr_last / lr_first)^(e / epochs).
    x1, x2, y = np.array([0.0]), np.array([0.0]), np.array([-1.0])
    epochs = 20
    _, hist = oracle.linreg_sgd(x1, x2, y, np.zeros(epochs, np.int32), [0.0, 0.0, 0.0, 0.0], 1, epochs, 1e-3, 1e-5)
    residual = np.sqrt(hist)
    lr = (1.0 - residual[1:] / residual[:-1]) / 2.0
    want = 1e-3 * (1e-5 / 1e-3) ** (np.arange(epochs - 1) / epochs)
    np.testing.assert_allclose(lr, want, rtol=1e-9)


def test_sgd_recovers_true_parameters_without_noise(oracle):
    x1, x2, y = linreg.synthetic_data(4096, seed=3, noise=0.0)
    rng = np.random.default_rng(0)
    batch, epochs = 256, 4000
    rows = rng.integers(0, 4096, batch * epochs).astype(np.int32)
    p, hist = oracle.linreg_sgd(x1, x2, y, rows, linreg.INITIAL_PARAMS, batch, epochs, 1e-4, 1e-5)
    assert hist[-1] < 1e-3 * hist[0]
    # a, b, c settle quickly; the offset d is the flat direction of this loss and is still on its way
    np.testing.assert_allclose(p[:3], linreg.TRUE_PARAMS[:3], atol=0.05)
    assert 0.1 < p[3] < linreg.TRUE_PARAMS[3] + 0.05


def test_gradient_matches_reverse_mode_autodiff(oracle):
    """The summed loss sum_i ((x1 - a)^2 + b (x2 - c)^2 + d - y)^2 differentiated by PyTorch's autograd."""
    import torch

    x1, x2, y = linreg.synthetic_data(3000, seed=12, noise=0.3)
    for params in ([0.5, 1.5, -0.5, 0.2], [2.5, 1.8, -1.2, 0.5], [-3.0, 0.1, 4.0, -7.0]):
        p = torch.tensor(params, dtype=torch.float64, requires_grad=True)
        a, b, c, d = p
        loss = (((torch.tensor(x1) - a) ** 2 + b * (torch.tensor(x2) - c) ** 2 + d - torch.tensor(y)) ** 2).sum()
        loss.backward()
        out = oracle.linreg_gradient(x1, x2, y, params)
        np.testing.assert_allclose(out[:4], p.grad.numpy(), rtol=1e-11)
        np.testing.assert_allclose(out[4], float(loss.detach()), rtol=1e-12)
