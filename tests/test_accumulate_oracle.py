"""Pins the accumulation oracle (fp64 per-slot sums) against an independent numpy formulation."""
import numpy as np

from tests._metrics import chain_inputs


def _numpy_sums(oracle, inputs, slot, num_slots, dtype):
    g = oracle.chain_soa(inputs, dtype)[1:].astype(np.float64)  # six gradient rows
    ok = (slot >= 0) & (slot < num_slots)
    sums = np.stack([np.bincount(slot[ok], weights=g[k][ok], minlength=num_slots) for k in range(6)], axis=1)
    mass = np.stack([np.bincount(slot[ok], weights=np.abs(g[k][ok]), minlength=num_slots) for k in range(6)], axis=1)
    return sums, mass


def test_sums_match_numpy_bincount(oracle):
    n, num_slots = 50000, 37
    inputs = chain_inputs(n, seed=31)
    slot = np.random.default_rng(1).integers(-2, num_slots + 2, n).astype(np.int32)  # includes out-of-range entries
    for in_double, dtype in ((True, np.float64), (False, np.float32)):
        sums, mass = oracle.accumulate_chain(inputs, slot, num_slots, chain_in_double=in_double)
        want_sums, want_mass = _numpy_sums(oracle, inputs, slot, num_slots, dtype)
        assert np.allclose(sums, want_sums, rtol=1e-12, atol=1e-12 * want_mass.max())
        assert np.allclose(mass, want_mass, rtol=1e-12)


def test_counting_pattern_is_exact(oracle):
    """Every thread adds the same gradient to one slot: the sum is n times it
    (the shape of the reference's tests/test_parallel_gradient_accumulation.cu:94-99)."""
    n = 10000
    inputs = [np.full(n, v, np.float32) for v in (0.3, -0.7, 0.9, 0.25, 1.1, -0.4)]
    slot = np.zeros(n, np.int32)
    sums, _ = oracle.accumulate_chain(inputs, slot, 1, chain_in_double=True)
    _, g, _ = oracle.chain_one([float(a[0]) for a in inputs], np.float64)
    assert np.allclose(sums[0], n * g, rtol=1e-12)
