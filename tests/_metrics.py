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


FIELDS = ("cx", "cy", "log_sx", "log_sy", "theta", "r", "g", "b", "opacity")


def gradient_distribution(got, fp32_oracle, fp64, mass):
    """How an implementation's 9 x G gradients sit around the fp64 ones, field by field, beside the same figures
    for an independent fp32 evaluation (the fp32 oracle).  Errors are in units of `mass` (the sum of the
    magnitudes of the per-pixel terms behind a gradient: the scale of fp32 rounding in any summation order).

      median, p99      quantiles of |x - fp64| / mass over the Gaussians that reach a pixel, each Gaussian
                       weighted by its mass: "half (99 %) of the gradient mass sits in entries at least this
                       accurate".  (Unweighted, the upper quantiles are those of Gaussians hidden behind
                       others, whose few terms sit next to the 1e-4 stop, where two correct evaluations
                       differ by the whole term: 1 % of the Gaussians at 200 000, with next to no mass.)
      bias             sum (x - fp64) / sum mass: an error of one sign (terms left out, a list cut short)
      along_gradient   sum sign(fp64) (x - fp64) / sum mass: a factor on the gradients (a dropped 1/2, a wrong
                       constant) has the sign of the gradient even in fields whose gradients sum to nothing
      flat             fraction of the Gaussians with this gradient within 1e-4 relative
    """
    got, fp32_oracle, fp64, mass = (np.asarray(a, np.float64) for a in (got, fp32_oracle, fp64, mass))
    out = {}
    for row, field in enumerate(FIELDS):
        live = mass[row] > 0
        m, ref = mass[row][live], fp64[row][live]
        entry = {}
        for name, x in (("got", got[row][live]), ("fp32_oracle", fp32_oracle[row][live])):
            e = x - ref
            relative = np.abs(e) / m
            order = np.argsort(relative)
            share = np.cumsum(m[order]) / m.sum()
            entry[name] = {
                "median": float(relative[order][np.searchsorted(share, 0.5)]),
                "p99": float(relative[order][min(np.searchsorted(share, 0.99), relative.size - 1)]),
                "bias": float(e.sum() / m.sum()), "along_gradient": float((np.sign(ref) * e).sum() / m.sum()),
                "flat": float((np.abs(e) <= 1e-4 * np.abs(ref)).mean()),
            }
        out[field] = entry
    return out


def gradient_distribution_failures(figures, quantile_factor=1.5, bias_limit=2e-6, flat_slack=0.01, quantile_floor=1e-9):
    """What of gradient_distribution's figures is out of line: quantiles more than quantile_factor times the fp32
    oracle's own (plus quantile_floor: two fp32 evaluations of a few thousand Gaussians have medians of 1e-8 to 1e-7
    of the mass, below the 6e-8 an fp32 value resolves, and these vary by a factor of two from run to run with the
    order of the threads' sums), a bias (plain or along the gradient) beyond bias_limit, or fewer Gaussians within
    1e-4 relative than the fp32 oracle has (less flat_slack)."""
    failures = []
    for field, entry in figures.items():
        got, ref = entry["got"], entry["fp32_oracle"]
        for q in ("median", "p99"):
            if got[q] > quantile_factor * ref[q] + quantile_floor:
                failures.append("%s: %s of |error| / mass %.3g, the fp32 oracle's %.3g" % (field, q, got[q], ref[q]))
        for b in ("bias", "along_gradient"):
            if abs(got[b]) > bias_limit:
                failures.append("%s: %s %.3g (limit %.1g; the fp32 oracle's %.3g)" % (field, b, got[b], bias_limit, ref[b]))
        if got["flat"] < ref["flat"] - flat_slack:
            failures.append("%s: %.4f of the Gaussians within 1e-4 relative, the fp32 oracle %.4f" % (field, got["flat"], ref["flat"]))
    return failures
