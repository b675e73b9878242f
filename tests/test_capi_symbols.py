"""The C-ABI library loads without a GPU and exports exactly what include/xad_capi.h declares."""
import ctypes
import os
import re
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "xad_capi.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(xad_[a-z0-9_]+)\s*\(", text)))


def test_header_is_plain_c():
    src = '#include "xad_capi.h"\nint main(void) { return XAD_OK; }\n'
    proc = subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-pedantic", "-fsyntax-only", "-I", os.path.dirname(HEADER), "-x", "c", "-"],
                          input=src, capture_output=True, text=True)
    assert proc.returncode == 0, proc.stderr


def test_every_declared_entry_point_is_exported(xad):
    from xyz_autodiff_cuda_amd import _lib

    lib = ctypes.CDLL(_lib.LIB_PATH)
    names = declared_functions()
    assert len(names) >= 20
    for name in names:
        assert hasattr(lib, name), "declared in xad_capi.h but not exported: " + name
    # and the Python binding knows every one of them
    assert sorted(_lib.SIGNATURES) == names


def test_no_undeclared_xad_symbols_are_exported():
    from xyz_autodiff_cuda_amd import _lib

    out = subprocess.run(["nm", "-D", "--defined-only", _lib.LIB_PATH], capture_output=True, text=True, check=True).stdout
    exported = sorted(set(re.findall(r"\bT (xad_[a-z0-9_]+)$", out, flags=re.M)))
    assert exported == declared_functions()


def test_library_reports_errors_without_a_gpu(xad):
    lib = xad.load()
    assert lib.xad_abi_version() == 1
    status = lib.xad_host_chain_forward_backward_f32(4, *([None] * 13), 1)
    assert status == 1 and b"null" in lib.xad_last_error()
    status = lib.xad_adam_step_f32(4, 99, None, None, None, None, None, 0.9, 0.999, 1e-8, 1, None)
    assert status == 1 and b"rows" in lib.xad_last_error()


def test_product_does_not_reference_the_oracle():
    """Nothing under the package or include/ may import, link or call the oracle."""
    for base in ("xyz_autodiff_cuda_amd", "include"):
        for dirpath, _, files in os.walk(os.path.join(ROOT, base)):
            if os.path.basename(dirpath) == "build":
                continue
            for f in files:
                if f.endswith((".py", ".hip", ".cuh", ".h")):
                    text = open(os.path.join(dirpath, f), errors="replace").read()
                    assert "oracle" not in text.lower(), os.path.join(dirpath, f)
