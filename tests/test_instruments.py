"""The measurement library (instruments/) is separate from the product: it loads without a GPU, exports
exactly what instruments/xad_instruments.h declares, and the product neither declares nor loads it."""
import ctypes
import os
import re
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "instruments", "xad_instruments.h")


def _declared():
    text = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    return sorted(set(re.findall(r"\b(xadi_[a-z0-9_]+)\s*\(", text)))


def test_header_is_plain_c_and_matches_the_exports():
    import instruments

    src = '#include "xad_instruments.h"\nint main(void) { return 0; }\n'
    proc = subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-pedantic", "-fsyntax-only", "-I", os.path.dirname(HEADER), "-x", "c", "-"],
                          input=src, capture_output=True, text=True)
    assert proc.returncode == 0, proc.stderr
    out = subprocess.run(["nm", "-D", "--defined-only", instruments.LIB_PATH], capture_output=True, text=True, check=True).stdout
    exported = sorted(set(re.findall(r"\bT (\w+)$", out, flags=re.M)))
    assert exported == _declared() == sorted(instruments.SIGNATURES)
    lib = instruments.load()
    assert lib.xadi_lds_atomic_cycles(9, 0, ctypes.byref(ctypes.c_double())) != 0 and b"element" in lib.xadi_last_error()


def test_the_product_does_not_know_the_instruments():
    header = open(os.path.join(ROOT, "include", "xad_capi.h")).read()
    assert "xadi_" not in header and "probe" not in header.lower()
    for dirpath, _, files in os.walk(os.path.join(ROOT, "xyz_autodiff_cuda_amd")):
        if os.path.basename(dirpath) == "build":
            continue
        for f in files:
            if f.endswith((".py", ".cpp", ".h")) or (f.endswith((".hip", ".cuh")) and f != "chain_device.cuh"):
                text = open(os.path.join(dirpath, f), errors="replace").read()
                assert "instruments" not in text and "xadi_" not in text, os.path.join(dirpath, f)
