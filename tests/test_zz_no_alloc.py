"""The allocation-free SGD entry point against the allocating one, through the C ABI.

xad_linreg_sgd_f64_static keeps the gradient sums of a step in an array inside
the library's device image instead of allocating them.  Both entry points run
the same kernels on the same rows, so their results differ only by the order
of the fp64 sums inside a step (1e-16 relative per step; the iteration
contracts): parameters and loss history must agree to 1e-9 relative, the bound
the trajectory test of the allocating entry point uses against the CPU
restatement, which is checked here as well.

Two calls in a row, the second on a smaller problem (fewer rows, a smaller
batch, fewer steps): the second must not see anything the first left in the
shared array.  Collected last on purpose: a failure here must not hide other
tests from `pytest -x`.
"""
import numpy as np
import pytest

from xyz_autodiff_cuda_amd import linreg

pytestmark = pytest.mark.gpu


def _device(gpu, *arrays):
    import torch

    return [torch.from_numpy(np.ascontiguousarray(a)).to(gpu) for a in arrays]


def _run(gpu, data, batch, epochs, seed, static):
    import torch

    params = torch.tensor(linreg.INITIAL_PARAMS, dtype=torch.float64, device=gpu)
    history = torch.full((epochs,), -1.0, dtype=torch.float64, device=gpu)
    linreg.sgd(*data, params, batch, epochs, 1e-4, 1e-6, seed=seed, history=history, static_scratch=static)
    torch.cuda.synchronize()  # the static entry point only queues the work
    return params.cpu().numpy(), history.cpu().numpy()


def test_static_scratch_matches_allocating_entry_point_twice(gpu, oracle):
    import torch

    cases = [(100_000, 8192, 200, 5), (30_000, 1000, 40, 11)]  # rows, batch, steps, seed: the second is smaller
    for total, batch, epochs, seed in cases:
        x1, x2, y = linreg.synthetic_data(total, seed=6)
        data = _device(gpu, x1, x2, y)
        got_p, got_h = _run(gpu, data, batch, epochs, seed, static=True)
        want_p, want_h = _run(gpu, data, batch, epochs, seed, static=False)
        np.testing.assert_allclose(got_p, want_p, rtol=1e-9, atol=1e-10)
        np.testing.assert_allclose(got_h, want_h, rtol=1e-9)
        rows = np.concatenate([linreg.batch_rows(seed, e, batch, total) for e in range(epochs)])
        ref_p, ref_h = oracle.linreg_sgd(x1, x2, y, rows, linreg.INITIAL_PARAMS, batch, epochs, 1e-4, 1e-6)
        np.testing.assert_allclose(got_p, ref_p, rtol=1e-9, atol=1e-10)
        np.testing.assert_allclose(got_h, ref_h, rtol=1e-9)
        assert got_h[-1] < got_h[0]


def test_static_entry_point_allocates_nothing(gpu):
    """Two views of the device that see raw HIP allocations (PyTorch's own counters only see PyTorch's):
    the free memory of the device around a synchronised call, and a stream capture in the mode in which
    hipMalloc, hipFree and a wait for the stream are errors; the recorded call, replayed twice with ordinary
    work in between, must give what the allocating entry point gives."""
    import torch

    total, batch, epochs, seed = 40_000, 2048, 30, 9
    x1, x2, y = linreg.synthetic_data(total, seed=4)
    data = _device(gpu, x1, x2, y)
    want_p, want_h = _run(gpu, data, batch, epochs, seed, static=False)
    params = torch.tensor(linreg.INITIAL_PARAMS, dtype=torch.float64, device=gpu)
    start = params.clone()
    history = torch.empty(epochs, dtype=torch.float64, device=gpu)
    linreg.sgd(*data, params, batch, epochs, 1e-4, 1e-6, seed=seed, history=history, static_scratch=True)  # looks the array up
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info(gpu)[0]
    params.copy_(start)
    linreg.sgd(*data, params, batch, epochs, 1e-4, 1e-6, seed=seed, history=history, static_scratch=True)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info(gpu)[0] == free_before
    np.testing.assert_allclose(params.cpu().numpy(), want_p, rtol=1e-9, atol=1e-10)

    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    params.copy_(start)
    torch.cuda.synchronize()
    with torch.cuda.graph(graph, stream=stream, capture_error_mode="global"):
        linreg.sgd(*data, params, batch, epochs, 1e-4, 1e-6, seed=seed, history=history, static_scratch=True)
    torch.cuda.synchronize()
    for replay in range(2):
        params.copy_(start)
        history.fill_(-1.0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        np.testing.assert_allclose(params.cpu().numpy(), want_p, rtol=1e-9, atol=1e-10, err_msg="replay %d" % replay)
        np.testing.assert_allclose(history.cpu().numpy(), want_h, rtol=1e-9, err_msg="replay %d" % replay)


def test_static_scratch_starts_from_zero_after_an_unfinished_looking_state(gpu):
    # zero steps queue only the clearing kernel and leave params alone; a following run is unaffected
    import torch

    x1, x2, y = linreg.synthetic_data(5000, seed=2)
    data = _device(gpu, x1, x2, y)
    params = torch.tensor(linreg.INITIAL_PARAMS, dtype=torch.float64, device=gpu)
    linreg.sgd(*data, params, 512, 0, static_scratch=True)
    torch.cuda.synchronize()
    assert params.cpu().tolist() == list(linreg.INITIAL_PARAMS)
    a = _run(gpu, data, 512, 25, 3, static=True)
    b = _run(gpu, data, 512, 25, 3, static=False)
    np.testing.assert_allclose(a[0], b[0], rtol=1e-9, atol=1e-10)
    np.testing.assert_allclose(a[1], b[1], rtol=1e-9)


def test_static_scratch_rejects_bad_sizes(gpu, xad):
    import torch

    x = torch.zeros(4, dtype=torch.float64, device=gpu)
    with pytest.raises(xad.XadError, match="steps exceed"):
        linreg.sgd(x, x, x, x.clone(), batch=2, epochs=(1 << 20) + 1, static_scratch=True,
                   history=torch.empty((1 << 20) + 1, dtype=torch.float64, device=gpu))
    with pytest.raises(xad.XadError):
        linreg.sgd(x, x, x, x.clone(), batch=0, epochs=1, static_scratch=True)
