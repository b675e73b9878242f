"""Per-op access to the oracle: (outputs, input gradients) of one op logic, by name.

Names and operand shapes are those of tests/_native.py LOGICS, so a test can put
the library's templates and the oracle side by side.
"""
import numpy as np


def _arr(x, dtype):
    return np.ascontiguousarray(np.asarray(x, dtype=dtype).ravel())


def evaluate(oracle, name, operands, constants=(), upstream=None, dtype=np.float64):
    name = name.split("@")[0]  # "<logic>@<size>" is the same logic at another operand size
    dt = np.dtype(dtype)
    ops = [_arr(o, dt) for o in operands]
    k = _arr(constants, dt)
    z = lambda n: np.zeros(n, dt)

    def unary(fwd, bwd_args, n_out, fwd_args=None):
        y = z(n_out)
        oracle.call(fwd, dt, *(fwd_args if fwd_args is not None else (ops[0].size, ops[0])), y)
        g = _arr(np.ones(n_out) if upstream is None else upstream, dt)
        gx = z(ops[0].size)
        oracle.call(bwd_args[0], dt, *bwd_args[1](y, g), gx)
        return y, gx

    n = ops[0].size
    if name in ("exp", "sin", "cos", "sigmoid", "squared"):
        return unary(name + "_fwd", (name + "_bwd", lambda y, g: (n, ops[0], g)), n)
    if name == "neg":
        return unary("neg_fwd", ("neg_bwd", lambda y, g: (n, g)), n)
    if name == "sum":
        return unary("sum_fwd", ("sum_bwd", lambda y, g: (n, g)), 1)
    if name == "l1_norm":
        return unary("l1_fwd", ("l1_bwd", lambda y, g: (n, ops[0], g)), 1)
    if name == "l2_norm":
        return unary("l2_fwd", ("l2_bwd", lambda y, g: (n, ops[0], y, g)), 1)
    if name in ("add_constant", "sub_constant", "mul_constant", "div_constant"):
        kind = ["add_constant", "sub_constant", "mul_constant", "div_constant"].index(name)
        c = float(k[0])
        return unary("constant_fwd", ("constant_bwd", lambda y, g: (kind, n, c, g)), n, fwd_args=(kind, n, ops[0], c))
    if name in ("const_add", "const_sub"):
        # x +- k[i]: the binary rule with a constant second operand; only the first gradient is kept
        kind = 0 if name == "const_add" else 1
        y = z(n)
        oracle.call("binary_fwd", dt, kind, n, ops[0], k, y)
        g = _arr(np.ones(n) if upstream is None else upstream, dt)
        ga, gb = z(n), z(n)
        oracle.call("binary_bwd", dt, kind, n, ops[0], k, g, ga, gb)
        return y, ga
    if name == "sym_matrix2_inv":
        return unary("sym_matrix2_inv_fwd", ("sym_matrix2_inv_bwd", lambda y, g: (ops[0], g)), 3, fwd_args=(ops[0],))
    if name == "quaternion_to_rotation_matrix":
        return unary("quat_to_rot_fwd", ("quat_to_rot_bwd", lambda y, g: (ops[0], g)), 9, fwd_args=(ops[0],))
    if name == "matrix_to_covariance_3param":
        return unary("m_to_cov3_fwd", ("m_to_cov3_bwd", lambda y, g: (ops[0], g)), 3, fwd_args=(ops[0],))
    if name == "broadcast_logic":
        # include/xyz_autodiff/operations/unary/broadcast_logic.cuh:15-35 of the reference: copies, then the sum of gradients
        g = _arr(np.ones(4) if upstream is None else upstream, dt)
        return np.full(4, ops[0][0], dt), np.array([g.sum(dtype=dt)], dt)
    if name in ("add", "sub", "mul", "div"):
        kind = ["add", "sub", "mul", "div"].index(name)
        y = z(n)
        oracle.call("binary_fwd", dt, kind, n, ops[0], ops[1], y)
        g = _arr(np.ones(n) if upstream is None else upstream, dt)
        ga, gb = z(n), z(n)
        oracle.call("binary_bwd", dt, kind, n, ops[0], ops[1], g, ga, gb)
        return y, np.concatenate([ga, gb])
    if name in ("matmul_2x2", "matmul_3x3", "matvec_2x3", "vecmat_3x2"):
        ra, ca, cb = {"matmul_2x2": (2, 2, 2), "matmul_3x3": (3, 3, 3), "matvec_2x3": (2, 3, 1), "vecmat_3x2": (1, 3, 2)}[name]
        y = z(ra * cb)
        oracle.call("matmul_fwd", dt, ra, ca, cb, ops[0], ops[1], y)
        g = _arr(np.ones(ra * cb) if upstream is None else upstream, dt)
        ga, gb = z(ra * ca), z(ca * cb)
        oracle.call("matmul_bwd", dt, ra, ca, cb, ops[0], ops[1], g, ga, gb)
        return y, np.concatenate([ga, gb])
    if name in ("generate_covariance_matrix", "scale_rotation_to_covariance_3param"):
        base, n_out = {"generate_covariance_matrix": ("cov_matrix", 4), "scale_rotation_to_covariance_3param": ("scale_rot_to_cov3", 3)}[name]
        y = z(n_out)
        oracle.call(base + "_fwd", dt, ops[0], ops[1], y)
        g = _arr(np.ones(n_out) if upstream is None else upstream, dt)
        gs, gr = z(2), z(1)
        oracle.call(base + "_bwd", dt, ops[0], ops[1], g, gs, gr)
        return y, np.concatenate([gs, gr])
    if name == "mahalanobis_distance":
        y = z(1)
        oracle.call("mahalanobis_fwd", dt, ops[0], ops[1], y)
        g = _arr(np.ones(1) if upstream is None else upstream, dt)
        gd, gi = z(2), z(3)
        oracle.call("mahalanobis_bwd", dt, ops[0], ops[1], g, gd, gi)
        return y, np.concatenate([gd, gi])
    if name == "mahalanobis_distance_with_center":
        y = z(1)
        px, py = float(k[0]), float(k[1])
        oracle.call("mahalanobis_center_fwd", dt, px, py, ops[0], ops[1], y)
        g = _arr(np.ones(1) if upstream is None else upstream, dt)
        gc, gi = z(2), z(3)
        oracle.call("mahalanobis_center_bwd", dt, px, py, ops[0], ops[1], g, gc, gi)
        return y, np.concatenate([gc, gi])
    raise KeyError(name)


# Input ranges per logic, following the reference's gradient tests
# (tests/operation/unary/*_gradient.cu, tests/operation/binary/*_gradient.cu,
# examples/mini-gaussian-splatting/tests/*.cu): mostly [-2, 2]; positive and away
# from zero where the operation needs it.
def sample_inputs(name, rng):
    from tests._native import LOGICS

    _, sizes, n_const, _ = LOGICS[name]
    name = name.split("@")[0]
    lo, hi = -2.0, 2.0
    operands = [rng.uniform(lo, hi, s) for s in sizes]
    constants = rng.uniform(0.5, 2.0, n_const) * rng.choice([-1.0, 1.0], n_const) if n_const else np.zeros(0)
    if name == "div":
        operands[1] = rng.uniform(0.5, 2.0, sizes[1]) * rng.choice([-1.0, 1.0], sizes[1])
    if name == "sym_matrix2_inv":  # tests/operation/unary/test_sym_matrix2_inv.cu:61-68: [0.5, 3], kept positive definite
        a, c = rng.uniform(1.0, 3.0, 2)
        b = rng.uniform(-0.5, 0.5) * np.sqrt(a * c)
        operands = [np.array([a, b, c])]
    if name in ("l1_norm", "l2_norm"):  # away from the kink at zero
        operands = [rng.uniform(0.2, 2.0, sizes[0]) * rng.choice([-1.0, 1.0], sizes[0])]
    if name in ("generate_covariance_matrix", "scale_rotation_to_covariance_3param"):
        operands = [rng.uniform(0.3, 2.5, 2), rng.uniform(-np.pi, np.pi, 1)]
    if name in ("mahalanobis_distance", "mahalanobis_distance_with_center"):
        a, c = rng.uniform(0.5, 2.0, 2)
        operands = [rng.uniform(-2, 2, 2), np.array([a, rng.uniform(-0.4, 0.4) * np.sqrt(a * c), c])]
        constants = rng.uniform(-2, 2, n_const)
    if name == "quaternion_to_rotation_matrix":
        q = rng.normal(0, 1, 4)
        operands = [q / np.linalg.norm(q)]
    return operands, constants
