"""GPU parity of the per-thread forward+backward kernels, through the C ABI.

Tolerances (fp32): the forward value within 1e-5 (abs-or-rel, the reference
testers' measure) on every problem; gradients within 1e-5 wherever the
covariance is well conditioned and within 1e-5 x cond(Sigma) in general, against
both the fp32 and the fp64 oracle.  The fp32 oracle itself is only that close to
fp64 (tests/test_oracle_chain.py), so nothing tighter is meaningful.
"""
import numpy as np
import pytest

from tests._metrics import abs_or_rel, chain_closed_form, chain_inputs, covariance_condition

pytestmark = pytest.mark.gpu


def _run_gpu(inputs, gpu, offset=0, problems_per_lane=None):
    """problems_per_lane None: the library (one problem per lane); 1 or 4: the same kernel body with the
    lane-to-address mapping chosen, from the measurement library (instruments/)."""
    import torch

    import instruments
    from xyz_autodiff_cuda_amd import chain

    n = inputs[0].size
    dev = []
    for a in inputs:
        buf = torch.empty(n + offset, dtype=torch.float32, device=gpu)
        view = buf[offset:]
        view.copy_(torch.from_numpy(np.ascontiguousarray(a)))
        dev.append(view)
    outs = [torch.full((n + offset,), float("nan"), dtype=torch.float32, device=gpu)[offset:] for _ in range(7)]
    if problems_per_lane is None:
        chain.forward_backward(dev, outs)
    else:
        instruments.chain_with_layout(dev, outs, problems_per_lane)
    torch.cuda.synchronize()
    return np.stack([o.cpu().numpy() for o in outs])


def _check(got, inputs, oracle):
    ref32 = oracle.chain_soa(inputs, np.float32)
    ref64 = oracle.chain_soa(inputs, np.float64)
    kappa = covariance_condition(inputs[0], inputs[1])
    assert np.isfinite(got).all()
    for ref in (ref32, ref64):
        e = abs_or_rel(got, ref)
        assert e[0].max() < 1e-5
        assert e[:, kappa <= 7.4].max(initial=0.0) < 1e-5
        assert (e / np.maximum(1.0, kappa)).max() < 1e-5
    assert abs_or_rel(got, ref64).max() <= 2.0 * abs_or_rel(ref32, ref64).max()


@pytest.mark.parametrize("lanes", [None, 1, 4])
@pytest.mark.parametrize("n", [1, 3, 4, 5, 255, 256, 257, 1023, 1024, 1025, 4096, 100003])
def test_sizes_around_vector_and_block_edges(gpu, oracle, n, lanes):
    inputs = chain_inputs(n, seed=100 + n)
    _check(_run_gpu(inputs, gpu, problems_per_lane=lanes), inputs, oracle)


def test_one_million_problems(gpu, oracle):
    inputs = chain_inputs(1_000_000, seed=7)
    got = _run_gpu(inputs, gpu)
    _check(got, inputs, oracle)
    # independent closed form, fp64
    want, _ = chain_closed_form(inputs)
    kappa = covariance_condition(inputs[0], inputs[1])
    assert (abs_or_rel(got, want) / np.maximum(1.0, kappa)).max() < 1e-5


def test_both_lane_mappings_and_unaligned_buffers_agree_bitwise(gpu, oracle):
    inputs = chain_inputs(5003, seed=9)
    a = _run_gpu(inputs, gpu, offset=0, problems_per_lane=1)
    b = _run_gpu(inputs, gpu, offset=0, problems_per_lane=4)
    c = _run_gpu(inputs, gpu, offset=1, problems_per_lane=4)  # 4-byte aligned only: falls to 4-byte accesses
    assert np.array_equal(a, b)
    assert np.array_equal(a, c)


def test_store_policies_of_the_instrument_agree_bitwise(gpu, xad):
    """The store-policy instrument changes how results are stored, never what is stored."""
    import torch

    import instruments
    from xyz_autodiff_cuda_amd import chain

    n = 70_001
    ins = [torch.from_numpy(a).to(gpu) for a in chain_inputs(n, seed=12)]
    want = torch.stack(chain.forward_backward(ins))
    for policy in instruments.STORE_POLICIES:
        outs = [torch.full((n,), float("nan"), dtype=torch.float32, device=gpu) for _ in range(7)]
        instruments.chain_with_store_policy(ins, outs, policy)
        assert torch.equal(torch.stack(outs), want), policy
    with pytest.raises(instruments.InstrumentError, match="policy"):
        instruments.chain_with_store_policy(ins, outs, 7)
    copy = instruments.stream_copy(ins[0], torch.zeros_like(ins[0]))
    assert torch.equal(copy, ins[0])
    resources = instruments.chain_kernel_resources()
    assert resources["scratch_bytes"] == 0 and 0 < resources["vgprs"] <= 64 and resources["wavefronts_per_simd"] == 8


def test_device_matches_host_build_of_the_same_templates(gpu, xad):
    from xyz_autodiff_cuda_amd import chain

    inputs = chain_inputs(300000, seed=13)
    got = _run_gpu(inputs, gpu)
    host = np.stack(chain.host_forward_backward(inputs, np.float32))
    kappa = covariance_condition(inputs[0], inputs[1])
    e = abs_or_rel(got, host)
    assert e[0].max() < 1e-5
    assert (e / np.maximum(1.0, kappa)).max() < 1e-5


def test_empty(gpu, xad):
    import torch

    from xyz_autodiff_cuda_amd import chain

    z = [torch.empty(0, dtype=torch.float32, device=gpu) for _ in range(6)]
    outs = chain.forward_backward(z)
    assert all(o.numel() == 0 for o in outs)


def test_rejects_null_and_host_tensors(gpu, xad):
    import torch

    from xyz_autodiff_cuda_amd import _lib, chain

    with pytest.raises(TypeError):
        chain.forward_backward([torch.zeros(4)] * 6)
    lib = _lib.load()
    status = lib.xad_chain_forward_backward_f32(4, *([None] * 13), None)
    assert status != 0 and b"null" in lib.xad_last_error()


def test_full_size_finite_differences_property(gpu, oracle):
    """At the benchmark's full size (64 Mi problems) the oracle is too slow to
    run on everything: check all outputs are finite, a strided sample against the
    oracle, and the identity d w / d o = w (1 - sigmoid(o)) on every problem."""
    import torch

    from xyz_autodiff_cuda_amd import chain, rng

    n = 64 * 1024 * 1024
    ins = [torch.empty(n, dtype=torch.float32, device=gpu) for _ in range(6)]
    rng.chain_inputs_(ins, seed=1234)
    outs = chain.forward_backward(ins)
    torch.cuda.synchronize()
    for o in outs:
        assert bool(torch.isfinite(o).all())
    w, d_o = outs[0].double(), outs[4].double()
    sig = torch.sigmoid(ins[3].double())
    ident = (d_o - w * (1 - sig)).abs()
    assert float(ident.max()) < 1e-6
    idx = torch.arange(0, n, 997, device=gpu)
    sample = [t[idx].cpu().numpy() for t in ins]
    got = np.stack([o[idx].cpu().numpy() for o in outs])
    _check(got, sample, oracle)


def test_more_than_two_to_the_32_problems(gpu, oracle):
    """13 arrays of 2^32 + 4099 floats (223 GB) fit the 288 GB of one MI355X: indices beyond 32 bits and
    the seams between the launches such a call is split into.  Skipped where that much memory is not free."""
    import torch

    from xyz_autodiff_cuda_amd import chain, rng

    n = (1 << 32) + 4099
    torch.cuda.empty_cache()
    free, _ = torch.cuda.mem_get_info(gpu)
    if free < 13 * 4 * n + (4 << 30):
        pytest.skip("needs %.0f GB of free device memory, %.0f GB are free" % (13 * 4 * n / 1e9, free / 1e9))
    ins = [torch.empty(n, dtype=torch.float32, device=gpu) for _ in range(6)]
    rng.chain_inputs_(ins, seed=99)
    outs = [torch.empty(n, dtype=torch.float32, device=gpu) for _ in range(7)]
    # what a lane that is never launched would leave behind, at the places looked at below
    seam = (1 << 32) - (1 << 20)  # first problem of the second launch
    windows = [(0, 4096), ((1 << 31) - 2048, (1 << 31) + 2048), (seam - 2048, seam + 2048), ((1 << 32) - 2048, n)]
    for lo, hi in windows:
        for o in outs:
            o[lo:hi] = float("nan")
    chain.forward_backward(ins, outs)
    torch.cuda.synchronize()
    for lo, hi in windows:
        sample = [t[lo:hi].cpu().numpy() for t in ins]
        got = np.stack([o[lo:hi].cpu().numpy() for o in outs])
        _check(got, sample, oracle)
    # every problem: the identity d w / d o = w (1 - sigmoid(o)), in pieces that fit beside the arrays
    piece = 1 << 28
    for lo in range(0, n, piece):
        hi = min(n, lo + piece)
        w, d_o = outs[0][lo:hi].double(), outs[4][lo:hi].double()
        ident = (d_o - w * (1 - torch.sigmoid(ins[3][lo:hi].double()))).abs().max()
        assert float(ident) < 1e-6, (lo, float(ident))
    del ins, outs
    torch.cuda.empty_cache()
