"""Pins the oracle's per-op forward and backward rules (oracle/oracle_ops.inc).

Each rule is a restatement of one op-logic struct of the reference.  Before the
library is checked against them they are pinned by:
  - the forward values of independent numpy formulas,
  - central finite differences, in fp64, of the oracle's own forward (with a
    random upstream gradient, so a wrong sign, a dropped term or two swapped
    outputs changes the result),
  - textbook identities (a matrix times its inverse, orthonormal rotations).
"""
import zlib

import numpy as np
import pytest

from tests import _native, _oracle_ops
from tests._metrics import abs_or_rel

NAMES = sorted(_native.LOGICS)


def _numpy_forward(name, ops, k):
    name = name.split("@")[0]  # "<logic>@<size>": the same logic at another operand size
    a = ops[0]
    b = ops[1] if len(ops) > 1 else None
    if name == "exp": return np.exp(a)
    if name == "sin": return np.sin(a)
    if name == "cos": return np.cos(a)
    if name == "sigmoid": return 1 / (1 + np.exp(-a))
    if name == "neg": return -a
    if name == "squared": return a * a
    if name == "sum": return np.array([a.sum()])
    if name == "l1_norm": return np.array([np.abs(a).sum()])
    if name == "l2_norm": return np.array([np.sqrt((a * a).sum())])
    if name == "add_constant": return a + k[0]
    if name == "sub_constant": return a - k[0]
    if name == "mul_constant": return a * k[0]
    if name == "div_constant": return a / k[0]
    if name == "const_add": return a + k
    if name == "const_sub": return a - k
    if name == "sym_matrix2_inv":
        inv = np.linalg.inv(np.array([[a[0], a[1]], [a[1], a[2]]]))
        return np.array([inv[0, 0], inv[0, 1], inv[1, 1]])
    if name == "quaternion_to_rotation_matrix":
        x, y, z, w = a
        return np.array([1 - 2 * (y * y + z * z), 2 * (x * y - z * w), 2 * (x * z + y * w), 2 * (x * y + z * w), 1 - 2 * (x * x + z * z),
                         2 * (y * z - x * w), 2 * (x * z - y * w), 2 * (y * z + x * w), 1 - 2 * (x * x + y * y)])
    if name == "broadcast_logic": return np.full(4, a[0])
    if name == "add": return a + b
    if name == "sub": return a - b
    if name == "mul": return a * b
    if name == "div": return a / b
    if name == "matmul_2x2": return (a.reshape(2, 2) @ b.reshape(2, 2)).ravel()
    if name == "matmul_3x3": return (a.reshape(3, 3) @ b.reshape(3, 3)).ravel()
    if name == "matvec_2x3": return a.reshape(2, 3) @ b
    if name == "vecmat_3x2": return a @ b.reshape(3, 2)
    R = lambda t: np.array([[np.cos(t), -np.sin(t)], [np.sin(t), np.cos(t)]])
    if name == "generate_covariance_matrix": return (R(b[0]) @ np.diag(a)).ravel()
    if name == "matrix_to_covariance_3param":
        S = a.reshape(2, 2) @ a.reshape(2, 2).T
        return np.array([S[0, 0], S[0, 1], S[1, 1]])
    if name == "scale_rotation_to_covariance_3param":
        M = R(b[0]) @ np.diag(a)
        S = M @ M.T
        return np.array([S[0, 0], S[0, 1], S[1, 1]])
    if name == "mahalanobis_distance":
        A = np.array([[b[0], b[1]], [b[1], b[2]]])
        return np.array([a @ A @ a])
    if name == "mahalanobis_distance_with_center":
        A = np.array([[b[0], b[1]], [b[1], b[2]]])
        d = k - a
        return np.array([d @ A @ d])
    raise KeyError(name)


@pytest.mark.parametrize("name", NAMES)
def test_forward_matches_numpy_and_backward_matches_finite_differences(oracle, name):
    rng = np.random.default_rng(zlib.crc32(name.encode()))
    _, sizes, _, n_out = _native.LOGICS[name]
    for _ in range(25):
        ops, k = _oracle_ops.sample_inputs(name, rng)
        up = rng.uniform(-1.5, 1.5, n_out)
        y, g = _oracle_ops.evaluate(oracle, name, ops, k, up, np.float64)
        assert np.allclose(y, _numpy_forward(name, ops, k), rtol=1e-12, atol=1e-12), name
        flat = np.concatenate(ops)
        h = 1e-6
        fd = np.zeros_like(flat)
        for i in range(flat.size):
            hi, lo = flat.copy(), flat.copy()
            hi[i] += h
            lo[i] -= h
            split = lambda v: [v[sum(sizes[:j]):sum(sizes[:j + 1])] for j in range(len(sizes))]
            fd[i] = (up @ (_numpy_forward(name, split(hi), k) - _numpy_forward(name, split(lo), k))) / (2 * h)
        assert abs_or_rel(g, fd).max() < 1e-6, (name, g, fd)


def test_quirks_of_the_reference_rules(oracle):
    # determinant guard of the 2x2 inverse: |det| < 1e-8 is replaced by +1e-8 (both passes)
    y, g = _oracle_ops.evaluate(oracle, "sym_matrix2_inv", [np.array([1.0, 1.0, 1.0])])
    assert np.allclose(y, [1e8, -1e8, 1e8])
    assert np.isfinite(g).all()
    # L1: sign(0) = 0;  L2: no gradient at (numerically) zero norm
    _, g = _oracle_ops.evaluate(oracle, "l1_norm", [np.array([0.0, 2.0, -3.0, 0.0])])
    assert np.array_equal(g, [0.0, 1.0, -1.0, 0.0])
    _, g = _oracle_ops.evaluate(oracle, "l2_norm", [np.zeros(4)])
    assert np.array_equal(g, np.zeros(4))
    # identities: inverse of the covariance of a rotation by theta with scales s
    S, _ = _oracle_ops.evaluate(oracle, "scale_rotation_to_covariance_3param", [np.array([1.5, 0.4]), np.array([0.7])])
    inv, _ = _oracle_ops.evaluate(oracle, "sym_matrix2_inv", [S])
    prod = np.array([[S[0], S[1]], [S[1], S[2]]]) @ np.array([[inv[0], inv[1]], [inv[1], inv[2]]])
    assert np.allclose(prod, np.eye(2), atol=1e-12)
    Rm, _ = _oracle_ops.evaluate(oracle, "quaternion_to_rotation_matrix", [np.array([0.5, 0.5, 0.5, 0.5])])
    assert np.allclose(Rm.reshape(3, 3) @ Rm.reshape(3, 3).T, np.eye(3), atol=1e-12)


def _torch_forward(name, ops, k):
    """Every op written once more, as a differentiable PyTorch expression (fp64)."""
    import torch

    name = name.split("@")[0]
    x = ops[0]
    if name in ("exp", "sin", "cos", "sigmoid"):
        return getattr(torch, name)(x)
    if name == "neg":
        return -x
    if name == "squared":
        return x * x
    if name == "sum":
        return x.sum().reshape(1)
    if name == "l1_norm":
        return x.abs().sum().reshape(1)
    if name == "l2_norm":
        return (x * x).sum().sqrt().reshape(1)
    if name in ("add_constant", "const_add"):
        return x + k
    if name in ("sub_constant", "const_sub"):
        return x - k
    if name == "mul_constant":
        return x * k
    if name == "div_constant":
        return x / k
    if name == "sym_matrix2_inv":
        a, b, c = x
        return torch.stack([c, -b, a]) / (a * c - b * b)
    if name == "quaternion_to_rotation_matrix":
        qx, qy, qz, qw = x
        return torch.stack([1 - 2 * (qy * qy + qz * qz), 2 * (qx * qy - qw * qz), 2 * (qx * qz + qw * qy),
                            2 * (qx * qy + qw * qz), 1 - 2 * (qx * qx + qz * qz), 2 * (qy * qz - qw * qx),
                            2 * (qx * qz - qw * qy), 2 * (qy * qz + qw * qx), 1 - 2 * (qx * qx + qy * qy)])
    if name == "broadcast_logic":
        return x.expand(4)
    if name == "add":
        return x + ops[1]
    if name == "sub":
        return x - ops[1]
    if name == "mul":
        return x * ops[1]
    if name == "div":
        return x / ops[1]
    if name in ("matmul_2x2", "matmul_3x3", "matvec_2x3", "vecmat_3x2"):
        ra, ca, cb = {"matmul_2x2": (2, 2, 2), "matmul_3x3": (3, 3, 3), "matvec_2x3": (2, 3, 1), "vecmat_3x2": (1, 3, 2)}[name]
        return (x.reshape(ra, ca) @ ops[1].reshape(ca, cb)).reshape(-1)
    if name in ("generate_covariance_matrix", "matrix_to_covariance_3param", "scale_rotation_to_covariance_3param"):
        if name == "matrix_to_covariance_3param":
            m = x.reshape(2, 2)
        else:
            c, s = torch.cos(ops[1][0]), torch.sin(ops[1][0])
            m = torch.stack([torch.stack([c, -s]), torch.stack([s, c])]) @ torch.diag(x)
            if name == "generate_covariance_matrix":
                return m.reshape(-1)
        cov = m @ m.T
        return torch.stack([cov[0, 0], cov[0, 1], cov[1, 1]])
    if name in ("mahalanobis_distance", "mahalanobis_distance_with_center"):
        a, b, c = ops[1]
        d = x if name == "mahalanobis_distance" else k - x
        inv = torch.stack([torch.stack([a, b]), torch.stack([b, c])])
        return (d @ inv @ d).reshape(1)
    raise KeyError(name)


@pytest.mark.parametrize("name", NAMES)
def test_backward_matches_reverse_mode_autodiff_of_an_independent_statement(oracle, name):
    """Outputs to 1e-12 and input gradients to 1e-11 against PyTorch's autograd of _torch_forward:
    far tighter than central differences can be, and with no rule of the oracle retyped."""
    import torch

    rng = np.random.default_rng(zlib.crc32(("autograd" + name).encode()))
    _, _, _, n_out = _native.LOGICS[name]
    for _ in range(10):
        ops, k = _oracle_ops.sample_inputs(name, rng)
        up = rng.uniform(-1.5, 1.5, n_out)
        y, g = _oracle_ops.evaluate(oracle, name, ops, k, up, np.float64)
        t_ops = [torch.tensor(np.asarray(o, np.float64), requires_grad=True) for o in ops]
        t_k = torch.tensor(np.asarray(k, np.float64))
        if t_k.numel() == 1:
            t_k = t_k.reshape(())
        out = _torch_forward(name, t_ops, t_k)
        (out * torch.tensor(up)).sum().backward()
        want_g = np.concatenate([t.grad.numpy().ravel() if t.grad is not None else np.zeros(t.numel()) for t in t_ops])
        assert abs_or_rel(y, out.detach().numpy()).max() < 1e-12, (name, y, out)
        assert abs_or_rel(g, want_g).max() < 1e-11, (name, g, want_g)
