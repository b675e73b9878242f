"""Counter-based synthetic inputs: device fills and the host view of the bits."""
import numpy as np

from . import _lib


def _stream_ptr(stream, device):
    import torch

    s = stream if stream is not None else torch.cuda.current_stream(device)
    return s.cuda_stream


def uniform_(t, seed, stream_id, lo, hi, stream=None):
    """Fills float32 CUDA tensor `t` with U[lo, hi); element i depends only on (seed, stream_id, i)."""
    import torch

    assert t.is_cuda and t.dtype == torch.float32 and t.is_contiguous()
    with torch.cuda.device(t.device):
        st = _lib.load().xad_rng_uniform_f32(t.data_ptr(), t.numel(), seed, stream_id, lo, hi, _stream_ptr(stream, t.device))
    _lib.check(st, "xad_rng_uniform_f32")
    return t


def normal_(t, seed, stream_id, mean, stddev, stream=None):
    """Fills float32 CUDA tensor `t` with N(mean, stddev^2) by Box-Muller."""
    import torch

    assert t.is_cuda and t.dtype == torch.float32 and t.is_contiguous()
    with torch.cuda.device(t.device):
        st = _lib.load().xad_rng_normal_f32(t.data_ptr(), t.numel(), seed, stream_id, mean, stddev, _stream_ptr(stream, t.device))
    _lib.check(st, "xad_rng_normal_f32")
    return t


def host_bits(n, seed, stream_id, first=0):
    out = np.empty(n, dtype=np.uint64)
    _lib.check(_lib.load().xad_host_rng_bits(out.ctypes.data, n, seed, stream_id, first), "xad_host_rng_bits")
    return out


def host_uniform(n, seed, stream_id, lo, hi):
    out = np.empty(n, dtype=np.float32)
    _lib.check(_lib.load().xad_host_rng_uniform_f32(out.ctypes.data, n, seed, stream_id, lo, hi), "xad_host_rng_uniform_f32")
    return out


def chain_inputs_(tensors, seed):
    """Fills the six chain input tensors with the benchmark's distributions:
    sx, sy ~ U(-2, 1); theta ~ U(-pi, pi); o ~ N(0, 1); px, py ~ N(0, 4)."""
    sx, sy, theta, o, px, py = tensors
    uniform_(sx, seed, 0, -2.0, 1.0)
    uniform_(sy, seed, 1, -2.0, 1.0)
    uniform_(theta, seed, 2, -float(np.pi), float(np.pi))
    normal_(o, seed, 3, 0.0, 1.0)
    normal_(px, seed, 4, 0.0, 2.0)
    normal_(py, seed, 5, 0.0, 2.0)
    return tensors
