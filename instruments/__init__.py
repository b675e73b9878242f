"""ctypes binding of instruments/libxad_instruments.so (declared in instruments/xad_instruments.h).

Measurement only: bench.py, the profiling runs and the tests that check the instruments themselves
load this; the package xyz_autodiff_cuda_amd never does.
"""
import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libxad_instruments.so")

_vp, _sz, _int = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int
SIGNATURES = {
    "xadi_last_error": [],
    "xadi_source_digest": [],
    "xadi_chain_forward_backward_f32_layout": [_sz] + [_vp] * 13 + [_int, _vp],
    "xadi_chain_store_policy": [_int, _sz] + [_vp] * 13 + [_vp],
    "xadi_stream_copy_f32": [_sz, _vp, _vp, _vp],
    "xadi_copy_variant_f32": [_int, _sz, _vp, _vp, _vp],
    "xadi_chain_kernel_resources": [_vp],
    "xadi_lds_atomic_cycles": [_int, _int, ctypes.POINTER(ctypes.c_double)],
}

STORE_POLICIES = {"write_through": 0, "plain": 1, "non_temporal": 2}
LDS_PROBE_ELEMENTS = ("f32", "f64", "u32", "u64")
LDS_PROBE_PATTERNS = ("64_distinct", "one_address", "16_lanes_share", "8_lanes_per_address", "stride_6")

_lib = None


class InstrumentError(RuntimeError):
    pass


def load():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError("instruments/libxad_instruments.so is not built; run `python instruments/build.py`")
    try:  # PyTorch's HIP runtime first, so that the process has one
        import torch  # noqa: F401
    except ImportError:
        pass
    lib = ctypes.CDLL(LIB_PATH)
    for name, argtypes in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.argtypes = argtypes
        fn.restype = ctypes.c_char_p if name in ("xadi_last_error", "xadi_source_digest") else ctypes.c_int
    import importlib.util

    spec = importlib.util.spec_from_file_location("xad_instruments_build", os.path.join(HERE, "build.py"))
    build = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(build)
    if lib.xadi_source_digest().decode() != build.source_digest():
        raise ImportError("instruments/libxad_instruments.so is older than its sources; run `python instruments/build.py`")
    _lib = lib
    return lib


def _check(status, what):
    if status != 0:
        raise InstrumentError("%s failed with status %d: %s" % (what, status, load().xadi_last_error().decode("utf-8", "replace")))


def _chain_args(inputs, outs):
    import torch

    n = inputs[0].numel()
    for t in list(inputs) + list(outs):
        if not (t.is_cuda and t.dtype == torch.float32 and t.is_contiguous() and t.numel() == n):
            raise ValueError("expected contiguous float32 CUDA tensors of one length")
    if len(inputs) != 6 or len(outs) != 7:
        raise ValueError("expected 6 inputs and 7 outputs")
    return n, [t.data_ptr() for t in inputs] + [t.data_ptr() for t in outs]


def chain_with_layout(inputs, outs, problems_per_lane, stream=None):
    """The chain kernel with 1 or 4 problems per lane (4- or 16-byte accesses); fills `outs`."""
    import torch

    n, ptrs = _chain_args(inputs, outs)
    s = stream if stream is not None else torch.cuda.current_stream(inputs[0].device)
    with torch.cuda.device(inputs[0].device):
        _check(load().xadi_chain_forward_backward_f32_layout(n, *ptrs, int(problems_per_lane), s.cuda_stream),
               "xadi_chain_forward_backward_f32_layout")
    return outs


def chain_with_store_policy(inputs, outs, policy, stream=None):
    """The chain kernel with write_through / plain / non_temporal stores; fills `outs`."""
    import torch

    n, ptrs = _chain_args(inputs, outs)
    if isinstance(policy, str):
        policy = STORE_POLICIES[policy]
    s = stream if stream is not None else torch.cuda.current_stream(inputs[0].device)
    with torch.cuda.device(inputs[0].device):
        _check(load().xadi_chain_store_policy(int(policy), n, *ptrs, s.cuda_stream), "xadi_chain_store_policy")
    return outs


def stream_copy(src, dst, stream=None):
    import torch

    assert src.is_cuda and dst.is_cuda and src.dtype == dst.dtype == torch.float32 and src.numel() == dst.numel()
    s = stream if stream is not None else torch.cuda.current_stream(src.device)
    with torch.cuda.device(src.device):
        _check(load().xadi_stream_copy_f32(src.numel(), src.data_ptr(), dst.data_ptr(), s.cuda_stream), "xadi_stream_copy_f32")
    return dst


COPY_VARIANTS = ("4B_x1_write_through", "4B_x8_write_through", "16B_x1_plain", "16B_x4_plain", "16B_x4_non_temporal",
                 "16B_read_4B_write_through_x2", "4B_x8_plain")


def copy_variant(src, dst, variant, stream=None):
    """dst = src by one of COPY_VARIANTS (name or index)."""
    import torch

    assert src.is_cuda and dst.is_cuda and src.dtype == dst.dtype == torch.float32 and src.numel() == dst.numel()
    if isinstance(variant, str):
        variant = COPY_VARIANTS.index(variant)
    s = stream if stream is not None else torch.cuda.current_stream(src.device)
    with torch.cuda.device(src.device):
        _check(load().xadi_copy_variant_f32(int(variant), src.numel(), src.data_ptr(), dst.data_ptr(), s.cuda_stream), "xadi_copy_variant_f32")
    return dst


def chain_kernel_resources():
    """{vgprs, scratch_bytes, lds_bytes, block_lanes, blocks_per_cu, wavefronts_per_simd} of the chain kernel."""
    out = (ctypes.c_int * 5)()
    _check(load().xadi_chain_kernel_resources(out), "xadi_chain_kernel_resources")
    vgprs, scratch, lds, lanes, blocks = list(out)
    return {"vgprs": vgprs, "scratch_bytes": scratch, "lds_bytes": lds, "block_lanes": lanes, "blocks_per_cu": blocks,
            "wavefronts_per_simd": blocks * (lanes // 64) // 4}


def lds_atomic_cycles():
    """Measures LDS atomic-add cost: {element: {pattern: cycles per wavefront instruction}}."""
    lib = load()
    out = {}
    for e, ename in enumerate(LDS_PROBE_ELEMENTS):
        out[ename] = {}
        for p, pname in enumerate(LDS_PROBE_PATTERNS):
            c = ctypes.c_double(0.0)
            _check(lib.xadi_lds_atomic_cycles(e, p, ctypes.byref(c)), "xadi_lds_atomic_cycles")
            out[ename][pname] = c.value
    return out
