"""GPU parity of parallel gradient accumulation, through the C ABI.

The truth is the oracle's fp64 sum of fp64 per-thread gradients.  A computed
sum may differ from it by (a) the rounding of the summation, bounded relative
to the mass of the terms, sum |g_i|, and (b) the fp32 error of each term, which
is 1e-5 x cond(Sigma_i) relative to |g_i| (tests/test_chain_gpu.py).  Hence

    |got - want| <= SUM_TOL * sum_i |g_i|  +  1e-5 * sum_i cond_i |g_i|

with SUM_TOL = 1e-4 for the staged strategies.  The naive strategy (one fp32
global atomic per thread, the reference's pattern) keeps an fp32 running sum of
up to n terms per element and is held to 1e-2.
"""
import numpy as np
import pytest

from tests._metrics import chain_inputs, covariance_condition

pytestmark = pytest.mark.gpu

STAGED = ["auto", "lds", "lds_f32", "wave_lds", "wave_lds_shallow", "lds_leaves"]
NAIVE = ["global_atomics", "global_leaves"]


def _zipf_slots(n, num_slots, seed, exponent=1.1):
    p = np.arange(1, num_slots + 1, dtype=np.float64) ** -exponent
    cdf = np.cumsum(p / p.sum())
    u = np.random.default_rng(seed).random(n)
    return np.minimum(np.searchsorted(cdf, u, side="right"), num_slots - 1).astype(np.int32)


def _reference(oracle, inputs, slot, num_slots):
    sums, mass = oracle.accumulate_chain(inputs, slot, num_slots, chain_in_double=True)
    g = oracle.chain_soa(inputs, np.float64)[1:]
    kappa = covariance_condition(inputs[0], inputs[1])
    ok = (slot >= 0) & (slot < num_slots)
    kmass = np.stack([np.bincount(slot[ok], weights=(np.maximum(1.0, kappa) * np.maximum(1.0, np.abs(g[k])))[ok], minlength=num_slots) for k in range(6)], axis=1)
    return sums, mass, kmass


def _run(gpu, inputs, slot, num_slots, strategy, prefill=0.0):
    import torch

    from xyz_autodiff_cuda_amd import accumulate

    dev_in = [torch.from_numpy(a).to(gpu) for a in inputs]
    dev_slot = torch.from_numpy(slot).to(gpu)
    grads = torch.full((num_slots, 6), prefill, dtype=torch.float32, device=gpu)
    accumulate.accumulate_chain_gradients(dev_in, dev_slot, grads, strategy)
    torch.cuda.synchronize()
    return grads.cpu().numpy().astype(np.float64)


def _assert_close(got, ref, sum_tol):
    sums, mass, kmass = ref
    bound = sum_tol * mass + 1e-5 * kmass + 1e-30
    excess = np.abs(got - sums) / bound
    assert excess.max() <= 1.0, (excess.max(), np.unravel_index(excess.argmax(), excess.shape))


@pytest.mark.parametrize("strategy", STAGED)
@pytest.mark.parametrize("num_slots", [1, 3, 64, 3072, 3073, 4096, 5001, 6144, 7000, 262144, 600000])
def test_staged_strategies_match_fp64_sums(gpu, oracle, strategy, num_slots):
    n = 1_000_003
    inputs = chain_inputs(n, seed=50 + num_slots % 97)
    slot = _zipf_slots(n, num_slots, seed=num_slots)
    ref = _reference(oracle, inputs, slot, num_slots)
    _assert_close(_run(gpu, inputs, slot, num_slots, strategy), ref, 1e-4)


@pytest.mark.parametrize("law", ["hot slots last", "uniform", "hot slots in the middle"])
@pytest.mark.parametrize("num_slots", [3073, 4096, 70000])
def test_auto_under_laws_whose_low_slots_are_not_the_hot_ones(gpu, oracle, law, num_slots):
    """Above one table's worth of slots `auto` gives the rows to the first slots, which suits a law that
    falls with the slot index; a block that sees another law claims its rows on first use instead.  The
    sums must be right either way (and with blocks deciding differently: the middle law mixes both)."""
    n = 1_000_003
    inputs = chain_inputs(n, seed=60 + num_slots % 89)
    zipf = _zipf_slots(n, num_slots, seed=num_slots + 1)
    if law == "hot slots last":
        slot = (num_slots - 1 - zipf).astype(np.int32)
    elif law == "uniform":
        slot = np.random.default_rng(num_slots).integers(0, num_slots, n).astype(np.int32)
    else:
        # the first half of the threads draw hot slots from the middle, the second half from the front
        slot = zipf.copy()
        slot[: n // 2] = (slot[: n // 2] + num_slots // 2) % num_slots
    ref = _reference(oracle, inputs, slot, num_slots)
    _assert_close(_run(gpu, inputs, slot, num_slots, "auto"), ref, 1e-4)


@pytest.mark.parametrize("strategy", NAIVE)
@pytest.mark.parametrize("num_slots", [3, 4096])
def test_naive_global_atomics(gpu, oracle, strategy, num_slots):
    n = 200_000
    inputs = chain_inputs(n, seed=77)
    slot = _zipf_slots(n, num_slots, seed=5)
    ref = _reference(oracle, inputs, slot, num_slots)
    _assert_close(_run(gpu, inputs, slot, num_slots, strategy), ref, 1e-2)


@pytest.mark.parametrize("num_slots", [10, 5001, 7000])  # one table; slots dealt to two tables; claimed rows
def test_adds_to_existing_values_and_ignores_out_of_range_slots(gpu, oracle, num_slots):
    n = 100_000
    inputs = chain_inputs(n, seed=3)
    slot = np.random.default_rng(9).integers(-3, num_slots + 3, n).astype(np.int32)
    slot[::50] = np.random.default_rng(10).choice([-1, -2**31, num_slots, 2**31 - 1], size=slot[::50].size)
    sums, mass, kmass = _reference(oracle, inputs, slot, num_slots)
    for strategy in ("auto", "lds_leaves"):
        got = _run(gpu, inputs, slot, num_slots, strategy, prefill=2.5)
        _assert_close(got - 2.5, (sums, mass + 2.5, kmass), 1e-4)


def test_uniform_slots_no_contention(gpu, oracle):
    n, num_slots = 300_000, 1000
    inputs = chain_inputs(n, seed=4)
    slot = (np.arange(n) % num_slots).astype(np.int32)
    ref = _reference(oracle, inputs, slot, num_slots)
    for strategy in ("auto", "wave_lds"):
        _assert_close(_run(gpu, inputs, slot, num_slots, strategy), ref, 1e-4)


def test_device_zipf_matches_its_law(gpu, xad):
    import torch

    from xyz_autodiff_cuda_amd import accumulate

    n, num_slots = 4_000_000, 64
    slot = torch.empty(n, dtype=torch.int32, device=gpu)
    accumulate.zipf_(slot, seed=1234, stream_id=10, num_slots=num_slots)
    counts = np.bincount(slot.cpu().numpy(), minlength=num_slots)
    assert counts.sum() == n and slot.min() >= 0 and slot.max() < num_slots
    p = np.arange(1, num_slots + 1, dtype=np.float64) ** -1.1
    p /= p.sum()
    # six binomial standard deviations per cell
    assert (np.abs(counts - n * p) <= 6 * np.sqrt(n * p * (1 - p)) + 1).all()


def test_rejects_bad_arguments(gpu, xad):
    import torch

    from xyz_autodiff_cuda_amd import _lib, accumulate

    t = [torch.zeros(8, device=gpu) for _ in range(6)]
    slot = torch.zeros(8, dtype=torch.int32, device=gpu)
    grads = torch.zeros(4, 6, device=gpu)
    with pytest.raises(_lib.XadError):
        accumulate.accumulate_chain_gradients(t, slot, grads, strategy=99)
    with pytest.raises(ValueError):
        accumulate.accumulate_chain_gradients(t, slot, torch.zeros(4, 5, device=gpu))


def test_lds_fp64_atomics_are_the_fast_ones(gpu, xad):
    """The measurement the fp64 LDS table rests on: a wavefront-wide ds_add_f64 to
    distinct addresses must be several times cheaper than a ds_add_f32."""
    import instruments

    cycles = instruments.lds_atomic_cycles()
    assert cycles["f64"]["64_distinct"] * 4 < cycles["f32"]["64_distinct"]
    assert cycles["f64"]["one_address"] > cycles["f64"]["64_distinct"]
