"""Per-thread forward+backward of the benchmark graph (GPU and host-core builds).

Mirrors the way the reference's tests drive a graph kernel: six leaf arrays in,
the root value and the six leaf gradients out (tests/test_dag_backward.cu:43-67
in xyz-autodiff-cuda; the graph itself is that of
examples/mini-gaussian-splatting/gaussian_splatting_kernel.cu:86-97).
"""
import numpy as np

from . import _lib

INPUT_NAMES = ("sx", "sy", "theta", "o", "px", "py")
OUTPUT_NAMES = ("w", "d_sx", "d_sy", "d_theta", "d_o", "d_px", "d_py")
BYTES_PER_EVAL = 4 * (len(INPUT_NAMES) + len(OUTPUT_NAMES))  # 24 read + 28 written


def _require_cuda_f32(t, name, n):
    import torch

    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise TypeError("%s must be a tensor on the GPU" % name)
    if t.dtype != torch.float32 or not t.is_contiguous() or t.numel() != n:
        raise ValueError("%s must be a contiguous float32 tensor of %d elements" % (name, n))


def forward_backward(inputs, outputs=None, stream=None):
    """Runs the graph for every problem on the GPU.

    inputs:  six float32 CUDA tensors (sx, sy, theta, o, px, py) of equal length n.
    outputs: optional seven preallocated float32 CUDA tensors; allocated if None.
    stream:  torch.cuda.Stream to launch on (default: the current stream).
    Returns the seven output tensors (w, d_sx, d_sy, d_theta, d_o, d_px, d_py).
    """
    import torch

    lib = _lib.load()
    if len(inputs) != 6:
        raise ValueError("expected 6 input arrays, got %d" % len(inputs))
    n = inputs[0].numel()
    for t, name in zip(inputs, INPUT_NAMES):
        _require_cuda_f32(t, name, n)
    if outputs is None:
        outputs = [torch.empty(n, dtype=torch.float32, device=inputs[0].device) for _ in OUTPUT_NAMES]
    if len(outputs) != 7:
        raise ValueError("expected 7 output arrays, got %d" % len(outputs))
    for t, name in zip(outputs, OUTPUT_NAMES):
        _require_cuda_f32(t, name, n)
    s = stream if stream is not None else torch.cuda.current_stream(inputs[0].device)
    ptrs = [t.data_ptr() for t in inputs] + [t.data_ptr() for t in outputs]
    with torch.cuda.device(inputs[0].device):
        status = lib.xad_chain_forward_backward_f32(n, *ptrs, s.cuda_stream)
    _lib.check(status, "xad_chain_forward_backward_f32")
    return outputs


def host_forward_backward(inputs, dtype=np.float32, num_threads=0):
    """The same templates compiled for the host cores; numpy in, numpy out."""
    lib = _lib.load()
    dtype = np.dtype(dtype)
    fn = {
        np.dtype(np.float32): lib.xad_host_chain_forward_backward_f32,
        np.dtype(np.float64): lib.xad_host_chain_forward_backward_f64,
    }[dtype]
    arrays = [np.ascontiguousarray(a, dtype=dtype) for a in inputs]
    if len(arrays) != 6:
        raise ValueError("expected 6 input arrays, got %d" % len(arrays))
    n = arrays[0].size
    if any(a.size != n for a in arrays):
        raise ValueError("input arrays differ in length")
    outs = [np.empty(n, dtype=dtype) for _ in OUTPUT_NAMES]
    status = fn(n, *[a.ctypes.data for a in arrays], *[a.ctypes.data for a in outs], int(num_threads))
    _lib.check(status, fn.__name__)
    return outs
