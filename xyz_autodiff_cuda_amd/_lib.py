"""ctypes binding of libxad_hip.so (declared in include/xad_capi.h).

The library is loaded from this directory only.  There is no fallback: if it
has not been built, importing any compute entry point raises.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libxad_hip.so")

XAD_OK = 0
XAD_ERR_INCOMPLETE = 5


class XadError(RuntimeError):
    """A C-ABI call returned a non-zero status."""


_lib = None

_f32p = ctypes.POINTER(ctypes.c_float)
_f64p = ctypes.POINTER(ctypes.c_double)
_i32p = ctypes.POINTER(ctypes.c_int32)
_u64p = ctypes.POINTER(ctypes.c_uint64)
_sz = ctypes.c_size_t
_u64 = ctypes.c_uint64
_vp = ctypes.c_void_p
_int = ctypes.c_int
_flt = ctypes.c_float

# name -> argument types; every function returns int unless listed in _RESTYPE.
SIGNATURES = {
    "xad_last_error": [],
    "xad_abi_version": [],
    "xad_source_digest": [],
    "xad_chain_forward_backward_f32": [_sz] + [_vp] * 13 + [_vp],
    "xad_host_chain_forward_backward_f32": [_sz] + [_vp] * 13 + [_int],
    "xad_host_chain_forward_backward_f64": [_sz] + [_vp] * 13 + [_int],
    "xad_accumulate_chain_gradients_f32": [_int, _sz] + [_vp] * 8 + [_int, _vp],
    "xad_splat_create": [_int, _int, _int, _sz, ctypes.POINTER(_vp)],
    "xad_splat_destroy": [_vp],
    "xad_splat_forward": [_vp, _vp, _vp, _vp, _vp],
    "xad_splat_step": [_vp, _vp, _vp, _vp, _vp, _vp, ctypes.POINTER(ctypes.c_double), _vp],
    "xad_splat_set_profiling": [_vp, _int],
    "xad_splat_set_depth_mode": [_vp, _int],
    "xad_splat_get_lists": [_vp, _vp, _vp, _vp, _sz],
    "xad_host_splat_step_f32": [_int, _int, _int, _vp, _vp, _vp, _vp, _vp, ctypes.POINTER(ctypes.c_double), ctypes.POINTER(_u64), _int],
    "xad_splat_get_stats": [_vp, ctypes.POINTER(_u64), ctypes.POINTER(ctypes.c_uint32), ctypes.POINTER(_flt)],
    "xad_adam_step_f32": [_sz, _int, _vp, _vp, _vp, _vp, ctypes.POINTER(_flt), _flt, _flt, _flt, _int, _vp],
    "xad_adam_step_gated_f32": [_sz, _int, _vp, _vp, _vp, _vp, ctypes.POINTER(_flt), _flt, _flt, _flt, _int, _vp, _vp, _vp],
    "xad_splat_overflow_word": [_vp, ctypes.POINTER(_vp)],
    "xad_depth_order_f32": [_sz, _vp, _vp, _vp, _vp],
    "xad_training_config_defaults": [_vp],
    "xad_training_config_parse": [_int, ctypes.POINTER(ctypes.c_char_p), _vp],
    "xad_training_config_validate": [_vp],
    "xad_training_usage": [],
    "xad_image_load": [ctypes.c_char_p, ctypes.POINTER(_int), ctypes.POINTER(_int), ctypes.POINTER(_f32p)],
    "xad_image_free": [_f32p],
    "xad_image_save": [ctypes.c_char_p, _int, _int, _vp],
    "xad_image_save_jpeg": [ctypes.c_char_p, _int, _int, _vp, _int],
    "xad_image_test_pattern": [_int, _int, _vp],
    "xad_trainer_create": [_vp, _int, _int, _vp, ctypes.POINTER(_vp)],
    "xad_trainer_destroy": [_vp],
    "xad_trainer_run": [_vp, _int, ctypes.POINTER(ctypes.c_double)],
    "xad_trainer_iteration": [_vp],
    "xad_trainer_repeated_iterations": [_vp],
    "xad_trainer_download_image": [_vp, _vp],
    "xad_trainer_get_state": [_vp, _vp, _vp, _vp, _vp],
    "xad_trainer_set_params": [_vp, _vp, _vp],
    "xad_trainer_save_checkpoint": [_vp, ctypes.c_char_p],
    "xad_trainer_load_checkpoint": [_vp, ctypes.c_char_p],
    "xad_linreg_gradient_f64": [_int, _sz, _sz, _vp, _vp, _vp, _vp, _vp, _vp, _vp],
    "xad_linreg_sgd_f64": [_sz, _vp, _vp, _vp, _vp, _int, _int, ctypes.c_double, ctypes.c_double, _u64, _vp, _vp],
    "xad_linreg_sgd_f64_static": [_sz, _vp, _vp, _vp, _vp, _int, _int, ctypes.c_double, ctypes.c_double, _u64, _vp, _vp],
    "xad_host_linreg_gradient_f64": [_sz, _sz, _vp, _vp, _vp, _vp, _vp, _vp],
    "xad_rng_zipf_i32": [_vp, _sz, _u64, _u64, _int, ctypes.c_double, _vp],
    "xad_rng_uniform_f32": [_vp, _sz, _u64, _u64, _flt, _flt, _vp],
    "xad_rng_normal_f32": [_vp, _sz, _u64, _u64, _flt, _flt, _vp],
    "xad_host_rng_bits": [_vp, _sz, _u64, _u64, _u64],
    "xad_host_rng_uniform_f32": [_vp, _sz, _u64, _u64, _flt, _flt],
}
_RESTYPE = {"xad_last_error": ctypes.c_char_p, "xad_source_digest": ctypes.c_char_p, "xad_training_usage": ctypes.c_char_p,
            "xad_training_config_defaults": None, "xad_image_free": None, "xad_trainer_destroy": None, "xad_splat_destroy": None,
            "xad_trainer_repeated_iterations": ctypes.c_longlong}


def load():
    """Returns the loaded library, loading it on first use."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            "libxad_hip.so is not built (expected at %s); run `python -m xyz_autodiff_cuda_amd.build`" % LIB_PATH
        )
    # PyTorch brings a HIP runtime of its own; whichever of the two libraries is loaded first decides which
    # runtime the process uses.  With PyTorch first there is one runtime, the one that owns the tensors'
    # memory; with this library first its kernels found no device once PyTorch had initialised its own.
    try:
        import torch  # noqa: F401
    except ImportError:
        pass
    lib = ctypes.CDLL(LIB_PATH)
    for name, argtypes in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.argtypes = argtypes
        fn.restype = _RESTYPE.get(name, ctypes.c_int)
    from . import build

    built_from = lib.xad_source_digest().decode()
    if built_from != build.source_digest():
        raise ImportError(
            "libxad_hip.so was built from other sources than the ones next to it (digest %s...); "
            "rebuild with `python -m xyz_autodiff_cuda_amd.build`" % built_from[:12]
        )
    _lib = lib
    return lib


def check(status, what):
    if status != XAD_OK:
        msg = load().xad_last_error().decode("utf-8", "replace")
        raise XadError("%s failed with status %d: %s" % (what, status, msg))
