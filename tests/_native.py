"""ctypes access to tests/native/libxad_api_tier.so (the API test tier)."""
import ctypes
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "native", "libxad_api_tier.so")

_lib = None

# logic ids of xad_test_eval_logic: name -> (id, operand sizes, constants, outputs)
LOGICS = {
    "exp": (0, (3,), 0, 3), "sin": (1, (3,), 0, 3), "cos": (2, (3,), 0, 3), "sigmoid": (3, (3,), 0, 3),
    "neg": (4, (3,), 0, 3), "squared": (5, (3,), 0, 3), "sum": (6, (4,), 0, 1), "l1_norm": (7, (4,), 0, 1),
    "l2_norm": (8, (4,), 0, 1), "add_constant": (9, (3,), 1, 3), "sub_constant": (10, (3,), 1, 3),
    "mul_constant": (11, (3,), 1, 3), "div_constant": (12, (3,), 1, 3), "const_add": (13, (3,), 3, 3),
    "const_sub": (14, (3,), 3, 3), "sym_matrix2_inv": (15, (3,), 0, 3), "quaternion_to_rotation_matrix": (16, (4,), 0, 9),
    "broadcast_logic": (17, (1,), 0, 4), "add": (18, (3, 3), 0, 3), "sub": (19, (3, 3), 0, 3), "mul": (20, (3, 3), 0, 3),
    "div": (21, (3, 3), 0, 3), "matmul_2x2": (22, (4, 4), 0, 4), "matmul_3x3": (23, (9, 9), 0, 9),
    "matvec_2x3": (24, (6, 3), 0, 2), "vecmat_3x2": (25, (3, 6), 0, 2), "generate_covariance_matrix": (26, (2, 1), 0, 4),
    "matrix_to_covariance_3param": (27, (4,), 0, 3), "scale_rotation_to_covariance_3param": (28, (2, 1), 0, 3),
    "mahalanobis_distance": (29, (2, 3), 0, 1), "mahalanobis_distance_with_center": (30, (2, 3), 2, 1),
    # "<logic>@<size>": the same logic at another operand size
    "exp@1": (31, (1,), 0, 1), "exp@20": (32, (20,), 0, 20), "sigmoid@1": (33, (1,), 0, 1), "sigmoid@20": (34, (20,), 0, 20),
    "mul@1": (35, (1, 1), 0, 1), "mul@5": (36, (5, 5), 0, 5), "add@5": (37, (5, 5), 0, 5),
}


def load():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError("tests/native/libxad_api_tier.so is not built; run `python tests/native/build.py`")
        try:  # PyTorch's HIP runtime first, so that the process has one (see xyz_autodiff_cuda_amd/_lib.py)
            import torch  # noqa: F401
        except ImportError:
            pass
        lib = ctypes.CDLL(LIB_PATH)
        lib.xad_test_source_digest.restype = ctypes.c_char_p
        import importlib.util

        spec = importlib.util.spec_from_file_location("xad_native_build", os.path.join(HERE, "native", "build.py"))
        build = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(build)
        if lib.xad_test_source_digest().decode() != build.source_digest():
            raise ImportError("tests/native/libxad_api_tier.so is older than its sources; run `python tests/native/build.py`")
        _lib = lib
    return _lib


def run_case(case_id, device=False):
    lib = load()
    out = np.zeros(lib.xad_test_case_capacity(), np.float64)
    fn = lib.xad_test_run_case_device if device else lib.xad_test_run_case_host
    n = fn(ctypes.c_int(case_id), out.ctypes.data_as(ctypes.c_void_p))
    assert n >= 0, "case %d failed with %d" % (case_id, n)
    return out[:n]


def eval_logic(name, operands, constants=(), upstream=None, dtype=np.float64, delta=1e-6, device=False):
    """Returns (outputs, analytic gradient, numerical gradient) of one op logic, the
    gradients concatenated over the operands."""
    logic_id, sizes, n_const, n_out = LOGICS[name]
    flat = np.concatenate([np.asarray(o, np.float64).ravel() for o in operands] + [np.asarray(constants, np.float64).ravel()])
    assert flat.size == sum(sizes) + n_const, (name, flat.size)
    up = np.ones(n_out) if upstream is None else np.asarray(upstream, np.float64)
    out = np.zeros(64, np.float64)
    n = load().xad_test_eval_logic(ctypes.c_int(1 if device else 0), ctypes.c_int(logic_id),
                                   ctypes.c_int(1 if np.dtype(dtype) == np.float64 else 0),
                                   flat.ctypes.data_as(ctypes.c_void_p), ctypes.c_int(flat.size), up.ctypes.data_as(ctypes.c_void_p),
                                   ctypes.c_int(up.size), ctypes.c_double(delta), out.ctypes.data_as(ctypes.c_void_p))
    n_in = sum(sizes)
    assert n == n_out + 2 * n_in, (name, n)
    return out[:n_out].copy(), out[n_out:n_out + n_in].copy(), out[n_out + n_in:n].copy()


def negligible_in_tile(fields, tiles, device=False):
    """fields (n, 6) float32: centre x, y, inverse covariance a, b, c, alpha0; tiles (n, 2) float32: the tiles' first
    pixels.  -> bool array: the entries the compositing kernels would leave out of that tile."""
    fields = np.ascontiguousarray(fields, np.float32)
    tiles = np.ascontiguousarray(tiles, np.float32)
    n = fields.shape[0]
    assert fields.shape == (n, 6) and tiles.shape == (n, 2)
    out = np.zeros(n, np.int32)
    fn = load().xad_test_negligible_in_tile
    fn.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]
    rc = fn(1 if device else 0, n, fields.ctypes.data, tiles.ctypes.data, out.ctypes.data)
    assert rc == 0, rc
    return out.astype(bool)


def parallel_accumulation(threads, block):
    out = np.zeros(3, np.float64)
    rc = load().xad_test_parallel_accumulation(ctypes.c_size_t(threads), ctypes.c_int(block), out.ctypes.data_as(ctypes.c_void_p))
    assert rc == 0
    return out


def managed_accumulation(threads):
    """Gradient sums of `threads` add_grad calls on hipMallocManaged memory: (float: 2 sums, double: 2 sums)."""
    out = np.zeros(4, np.float64)
    rc = load().xad_test_managed_accumulation(ctypes.c_size_t(threads), out.ctypes.data_as(ctypes.c_void_p))
    assert rc == 0
    return out


def shared_accumulation(blocks, threads):
    out = np.zeros(2 * blocks, np.float64)
    rc = load().xad_test_shared_accumulation(ctypes.c_int(blocks), ctypes.c_int(threads), out.ctypes.data_as(ctypes.c_void_p))
    assert rc == 0
    return out.reshape(blocks, 2)


HOST_TESTER_PATH = os.path.join(HERE, "native", "libxad_tester_host.so")


def run_tester_suite(device):
    """Runs every gradient-tester call of the reference's tests plus the testers' self-checks:
    in kernels (the HIP build) or on the calling thread (the g++ build).  Returns
    (rows, self_check_bits), a row = (citation, name, cases, failures, worst error, on_device)."""
    if device:
        lib, fn_name = load(), "xad_test_tester_suite_device"
    else:
        if not os.path.exists(HOST_TESTER_PATH):
            raise ImportError("tests/native/libxad_tester_host.so is not built; run `python tests/native/build.py`")
        lib, fn_name = ctypes.CDLL(HOST_TESTER_PATH), "xad_test_tester_suite_host"
        lib.xad_test_host_source_digest.restype = ctypes.c_char_p
        load()  # checks the digest of the directory once ...
        if lib.xad_test_host_source_digest() != _lib.xad_test_source_digest():  # ... which both libraries carry
            raise ImportError("tests/native/libxad_tester_host.so is older than its sources; run `python tests/native/build.py`")
    fn = getattr(lib, fn_name)
    fn.argtypes = [ctypes.c_char_p, ctypes.c_size_t, ctypes.POINTER(ctypes.c_uint)]
    text = ctypes.create_string_buffer(1 << 16)
    bits = ctypes.c_uint(0)
    count = fn(text, len(text), ctypes.byref(bits))
    assert count >= 0, text.value.decode()
    rows = []
    for line in text.value.decode().splitlines():
        citation, name, cases, failures, worst, on_device = line.split("|")
        rows.append((citation, name, int(cases), int(failures), float(worst), on_device == "1"))
    assert len(rows) == count
    return rows, bits.value
