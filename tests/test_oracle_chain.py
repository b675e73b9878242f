"""Pins the CPU oracle of the per-thread graph before anything is checked against it.

The reference cannot be built in this toolchain (its headers need the CUDA
runtime header), so the restatement in oracle/ is pinned by:
  1. the one evaluation by the reference's own templates recorded in
     tests/golden/chain_reference_vector.json (fp32 and fp64, 9 digits);
  2. an independent closed form of the whole graph (no matrix inverse, no
     per-op rules) in fp64;
  3. central finite differences of the oracle's own forward value in fp64;
  4. the parameter sets the reference uses for its end-to-end gradient test
     (examples/mini-gaussian-splatting/tests/test_mini_gaussian_splatting_gradient.cu:235-303).
A dropped term, a sign error or a swapped index in any backward rule fails 2 and 3.
"""
import json
import os

import numpy as np
import pytest

from tests._metrics import abs_or_rel, chain_closed_form, chain_inputs

HERE = os.path.dirname(os.path.abspath(__file__))
ORDER = ("d_sx", "d_sy", "d_theta", "d_o", "d_px", "d_py")


def test_matches_recorded_reference_evaluation(oracle):
    with open(os.path.join(HERE, "golden", "chain_reference_vector.json")) as f:
        gold = json.load(f)
    x = [gold["inputs"][k] for k in ("sx", "sy", "theta", "o", "px", "py")]
    for key, dtype, tol in (("fp32", np.float32, 2e-7), ("fp64", np.float64, 5e-9)):
        w, g, q = oracle.chain_one(x, dtype)
        want = gold[key]
        # recorded with 9 significant digits: half a unit of the last printed digit
        assert abs(w - want["w"]) <= tol * abs(want["w"]) + 1e-12
        assert abs(q - want["q"]) <= tol * abs(want["q"])
        for i, name in enumerate(ORDER):
            assert abs(g[i] - want[name]) <= tol * abs(want[name]) + 1e-12, (key, name, g[i], want[name])


def test_fp64_matches_closed_form(oracle):
    inputs = chain_inputs(20000, seed=11)
    got = oracle.chain_soa(inputs, np.float64)
    want, _ = chain_closed_form(inputs)
    err = abs_or_rel(got, want)
    # both are fp64; what is left is the conditioning of the 2x2 inverse (<= e^6)
    assert err.max() < 1e-9, err.max(axis=1)


def test_fp64_matches_central_differences(oracle):
    inputs = chain_inputs(300, seed=5)
    x = np.stack([a.astype(np.float64) for a in inputs], axis=1)
    h = 1e-6
    for row in x:
        _, g, _ = oracle.chain_one(row, np.float64)
        for k in range(6):
            hi, lo = row.copy(), row.copy()
            hi[k] += h
            lo[k] -= h
            fd = (oracle.chain_one(hi, np.float64)[0] - oracle.chain_one(lo, np.float64)[0]) / (2 * h)
            assert abs_or_rel(g[k], fd) < 1e-5, (row, k, g[k], fd)


# (centre, scale, rotation, opacity logit, query point) of SimpleValues,
# NegativeValues and LargerValues; scales there are used through exp().
REFERENCE_PARAMETER_SETS = [
    ((0.0, 0.0), (1.0, 0.5), 0.1, 0.8, (0.5, 0.3)),
    ((-1.0, -0.5), (0.8, 1.2), -0.3, 0.6, (-0.8, -0.2)),
    ((5.0, 3.0), (2.0, 1.5), 1.2, 0.9, (4.5, 2.8)),
]


@pytest.mark.parametrize("centre,scale,rot,opacity,query", REFERENCE_PARAMETER_SETS)
def test_reference_parameter_sets(oracle, centre, scale, rot, opacity, query):
    x = [scale[0], scale[1], rot, opacity, query[0] - centre[0], query[1] - centre[1]]
    w, g, q = oracle.chain_one(x, np.float64)
    want, q_cf = chain_closed_form([np.array([v]) for v in x])
    assert abs(q - q_cf[0]) < 1e-10 * max(1.0, abs(q_cf[0]))
    assert abs_or_rel(np.concatenate([[w], g]), want[:, 0]).max() < 1e-10


def test_fp32_error_is_conditioning_not_a_bug(oracle):
    """fp32 vs fp64 of the same formulas: tight where Sigma is well conditioned,
    growing with its condition number elsewhere.  Fixes the scale the fp32 parity
    tolerances are written against."""
    from tests._metrics import covariance_condition

    inputs = chain_inputs(200000, seed=3)
    e = abs_or_rel(oracle.chain_soa(inputs, np.float32), oracle.chain_soa(inputs, np.float64))
    kappa = covariance_condition(inputs[0], inputs[1])
    assert e[0].max() < 1e-5  # the value itself
    assert e[:, kappa <= 7.4].max(initial=0.0) < 1e-5  # e^(2*1): more than half of all problems
    assert (e / np.maximum(1.0, kappa)).max() < 1e-5


def test_fp64_matches_reverse_mode_autodiff_of_an_independent_statement(oracle):
    """w = sigmoid(o) exp(-p^T Sigma^-1 p / 2) with Sigma = R(theta) diag(exp(s))^2 R(theta)^T inverted by a
    library routine; the six gradients by PyTorch's autograd.  Nothing of the oracle's rules is retyped here."""
    import torch

    inputs = [np.asarray(a, np.float64) for a in chain_inputs(500, seed=77)]
    got = oracle.chain_soa(inputs, np.float64)
    sx, sy, theta, o, px, py = (torch.tensor(a, requires_grad=True) for a in inputs)
    c, s = torch.cos(theta), torch.sin(theta)
    rot = torch.stack([torch.stack([c, -s], -1), torch.stack([s, c], -1)], -2)
    sigma = rot @ torch.diag_embed(torch.exp(torch.stack([sx, sy], -1)) ** 2) @ rot.transpose(-1, -2)
    p = torch.stack([px, py], -1)
    q = torch.einsum("ni,nij,nj->n", p, torch.linalg.inv(sigma), p)
    w = torch.sigmoid(o) * torch.exp(-0.5 * q)
    w.sum().backward()
    want = np.stack([w.detach().numpy()] + [t.grad.numpy() for t in (sx, sy, theta, o, px, py)])
    # the inverse of an ill-conditioned Sigma carries cond(Sigma) ulps in either evaluation
    kappa = np.exp(2.0 * np.abs(inputs[0] - inputs[1]))
    assert (abs_or_rel(got, want) / kappa).max() < 1e-12
