"""Least-squares fit of y ~ (x1 - a)^2 + b (x2 - c)^2 + d by mini-batch SGD, fp64.

Mirrors examples/optimization/linear_regression_sgd.cu of xyz-autodiff-cuda:
`batch_gradient` is its gradient kernel (:86-123) over a real batch with the
squared loss, `sgd` its training loop (:186-229), `synthetic_data` its
generate_data (:43-66) with a counter-based generator in place of std::mt19937.
"""
import ctypes

import numpy as np

from . import _lib

GLOBAL_ATOMICS = 0
LDS_LEAVES = 1
WAVE_LDS = 2
STRATEGIES = {"global_atomics": GLOBAL_ATOMICS, "lds_leaves": LDS_LEAVES, "wave_lds": WAVE_LDS}

TRUE_PARAMS = (2.5, 1.8, -1.2, 0.7)  # linear_regression_sgd.cu:17-20
INITIAL_PARAMS = (0.0, 1.0, 0.0, 0.0)  # :173-176
BYTES_PER_SAMPLE = 24


def _check_samples(x1, x2, y):
    import torch

    for t in (x1, x2, y):
        if not (t.is_cuda and t.dtype == torch.float64 and t.is_contiguous() and t.dim() == 1 and t.numel() == x1.numel()):
            raise ValueError("x1, x2, y must be contiguous float64 CUDA vectors of one length")


def batch_gradient(x1, x2, y, params, rows=None, strategy=WAVE_LDS, out=None, stream=None):
    """Sums d loss/d(a, b, c, d) and the loss over the batch.

    x1, x2, y: float64 CUDA vectors; params: float64 CUDA tensor of 4; rows: optional int32 CUDA
    vector of sample rows (the batch); returns a float64 CUDA tensor of 5 (4 gradient sums, loss sum).
    """
    import torch

    lib = _lib.load()
    if isinstance(strategy, str):
        strategy = STRATEGIES[strategy]
    _check_samples(x1, x2, y)
    if not (params.is_cuda and params.dtype == torch.float64 and params.is_contiguous() and params.numel() == 4):
        raise ValueError("params must be a contiguous float64 CUDA tensor of 4 elements")
    if rows is not None and not (rows.is_cuda and rows.dtype == torch.int32 and rows.is_contiguous()):
        raise ValueError("rows must be a contiguous int32 CUDA tensor")
    if out is None:
        out = torch.empty(5, dtype=torch.float64, device=x1.device)
    n = rows.numel() if rows is not None else x1.numel()
    s = stream if stream is not None else torch.cuda.current_stream(x1.device)
    with torch.cuda.device(x1.device):
        st = lib.xad_linreg_gradient_f64(int(strategy), n, x1.numel(), x1.data_ptr(), x2.data_ptr(), y.data_ptr(),
                                         rows.data_ptr() if rows is not None else None, params.data_ptr(),
                                         out.data_ptr(), s.cuda_stream)
    _lib.check(st, "xad_linreg_gradient_f64")
    return out


def sgd(x1, x2, y, params, batch, epochs, lr_first=1e-4, lr_last=1e-6, seed=0, want_history=False, stream=None,
        history=None, static_scratch=False):
    """Runs `epochs` steps on the device, updating `params` in place; returns the loss history or None.

    Defaults are the reference's learning rates (linear_regression_sgd.cu:26-27).
    static_scratch=True calls xad_linreg_sgd_f64_static: no device allocation inside the call (pass
    `history`, a float64 CUDA tensor of `epochs` elements, to keep this wrapper from allocating one
    too), and the call only queues the work: synchronise the stream before reading the results.
    """
    import torch

    lib = _lib.load()
    _check_samples(x1, x2, y)
    if not (params.is_cuda and params.dtype == torch.float64 and params.is_contiguous() and params.numel() == 4):
        raise ValueError("params must be a contiguous float64 CUDA tensor of 4 elements")
    if history is not None:
        if not (history.is_cuda and history.dtype == torch.float64 and history.is_contiguous() and history.numel() >= epochs):
            raise ValueError("history must be a contiguous float64 CUDA tensor of at least `epochs` elements")
    elif want_history:
        history = torch.empty(epochs, dtype=torch.float64, device=x1.device)
    s = stream if stream is not None else torch.cuda.current_stream(x1.device)
    name = "xad_linreg_sgd_f64_static" if static_scratch else "xad_linreg_sgd_f64"
    with torch.cuda.device(x1.device):
        st = getattr(lib, name)(x1.numel(), x1.data_ptr(), x2.data_ptr(), y.data_ptr(), params.data_ptr(),
                                int(batch), int(epochs), float(lr_first), float(lr_last), int(seed),
                                history.data_ptr() if history is not None else None, s.cuda_stream)
    _lib.check(st, name)
    return history


def host_batch_gradient(x1, x2, y, params, rows=None):
    """The library's templates compiled for the host, one thread; numpy float64 in, array of 5 out."""
    lib = _lib.load()
    x1, x2, y = (np.ascontiguousarray(a, dtype=np.float64) for a in (x1, x2, y))
    params = np.ascontiguousarray(params, dtype=np.float64)
    if params.size != 4 or not (x1.shape == x2.shape == y.shape and x1.ndim == 1):
        raise ValueError("expected three float64 vectors of one length and 4 parameters")
    if rows is not None:
        rows = np.ascontiguousarray(rows, dtype=np.int32)
    n = rows.size if rows is not None else x1.size
    out = np.empty(5, dtype=np.float64)
    P = ctypes.c_void_p
    st = lib.xad_host_linreg_gradient_f64(n, x1.size, x1.ctypes.data_as(P), x2.ctypes.data_as(P), y.ctypes.data_as(P),
                                          rows.ctypes.data_as(P) if rows is not None else None,
                                          params.ctypes.data_as(P), out.ctypes.data_as(P))
    _lib.check(st, "xad_host_linreg_gradient_f64")
    return out


def batch_rows(seed, epoch, batch, total):
    """Rows that step `epoch` of `sgd` draws (host restatement of the draw, for checking)."""
    from . import rng

    bits = rng.host_bits(batch, seed, 0, first=epoch * batch)
    return (bits % np.uint64(total)).astype(np.int32)


def synthetic_data(total, seed=0, noise=0.5, params=TRUE_PARAMS):
    """x1, x2 uniform in [-5, 5), y = model(true params) + normal noise: numpy float64 arrays."""
    from . import rng

    a, b, c, d = params
    u1 = rng.host_bits(total, seed, 1)
    u2 = rng.host_bits(total, seed, 2)
    x1 = (u1 >> np.uint64(11)).astype(np.float64) * 2.0 ** -53 * 10.0 - 5.0
    x2 = (u2 >> np.uint64(11)).astype(np.float64) * 2.0 ** -53 * 10.0 - 5.0
    g = np.random.Generator(np.random.PCG64(seed)).standard_normal(total) * noise
    y = (x1 - a) ** 2 + b * (x2 - c) ** 2 + d + g
    return x1, x2, y
