"""Error measures shared by the parity tests."""
import numpy as np


def abs_or_rel(got, want):
    """min(|got-want|, |got-want| / |want|): the measure of the reference's own
    gradient testers (include/xyz_autodiff/testing/unary_gradient_tester.cuh:28-32
    in xyz-autodiff-cuda)."""
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    diff = np.abs(got - want)
    return np.minimum(diff, diff / (np.abs(want) + 1e-15))


def covariance_condition(sx, sy):
    """Condition number of Sigma = R diag(e^sx, e^sy)^2 R^T: e^(2 |sx - sy|).
    Inverting Sigma from its three entries loses that factor in relative accuracy,
    whatever the implementation; it scales the fp32 gradient tolerances."""
    return np.exp(2.0 * np.abs(np.asarray(sx, np.float64) - np.asarray(sy, np.float64)))


def chain_inputs(n, seed):
    """The benchmark's input distributions, drawn with numpy for CPU-side tests:
    sx, sy ~ U(-2, 1); theta ~ U(-pi, pi); o ~ N(0, 1); px, py ~ N(0, 4)."""
    rng = np.random.default_rng(seed)
    arrays = [
        rng.uniform(-2.0, 1.0, n),
        rng.uniform(-2.0, 1.0, n),
        rng.uniform(-np.pi, np.pi, n),
        rng.normal(0.0, 1.0, n),
        rng.normal(0.0, 2.0, n),
        rng.normal(0.0, 2.0, n),
    ]
    return [a.astype(np.float32) for a in arrays]


def chain_closed_form(inputs):
    """w and d w / d (sx, sy, theta, o, px, py) in fp64 from an independent
    derivation (no matrix inverse, no chain of op rules):
        u = R(theta)^T p,  q = u0^2 e^(-2 sx) + u1^2 e^(-2 sy),  w = sigmoid(o) e^(-q/2)
        dq/dsx = -2 u0^2 e^(-2 sx),  dq/dsy = -2 u1^2 e^(-2 sy)
        dq/dtheta = 2 u0 u1 (e^(-2 sx) - e^(-2 sy))
        dq/dp = 2 R diag(e^(-2 s)) u
        dw/dq = -w / 2,  dw/do = w (1 - sigmoid(o))
    """
    sx, sy, th, o, px, py = [np.asarray(a, np.float64) for a in inputs]
    c, s = np.cos(th), np.sin(th)
    u0 = c * px + s * py
    u1 = -s * px + c * py
    ex, ey = np.exp(-2 * sx), np.exp(-2 * sy)
    q = u0 * u0 * ex + u1 * u1 * ey
    sig = 1.0 / (1.0 + np.exp(-o))
    w = sig * np.exp(-0.5 * q)
    dq = [
        -2 * u0 * u0 * ex,
        -2 * u1 * u1 * ey,
        2 * u0 * u1 * (ex - ey),
        None,
        2 * (c * ex * u0 - s * ey * u1),
        2 * (s * ex * u0 + c * ey * u1),
    ]
    grads = [(-0.5 * w) * d if d is not None else w * (1 - sig) for d in dq]
    return np.stack([w] + grads), q
