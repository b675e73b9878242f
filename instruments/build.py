"""Builds instruments/libxad_instruments.so (see xad_instruments.h) for gfx950, in-tree.

    python instruments/build.py

Same compiler flags as the product library, so the kernels measured here are the code the
product launches.  Every symbol but the xadi_ entry points is hidden.
"""
import hashlib
import importlib.util
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
LIB = os.path.join(HERE, "libxad_instruments.so")
SOURCES = [os.path.join(HERE, "instruments.hip")]


def _product_build():
    spec = importlib.util.spec_from_file_location("xad_product_build", os.path.join(ROOT, "xyz_autodiff_cuda_amd", "build.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def source_digest():
    """SHA-256 over this directory's sources and the product sources they include."""
    product = _product_build()
    h = hashlib.sha256(product.source_digest().encode())
    for name in ("instruments.hip", "xad_instruments.h"):
        with open(os.path.join(HERE, name), "rb") as f:
            h.update(name.encode() + b"\0" + f.read() + b"\0")
    return h.hexdigest()


def build():
    product = _product_build()
    cmd = [product.HIPCC, *product.FLAGS, "-fvisibility=hidden", "-DXADI_SOURCE_DIGEST=\"%s\"" % source_digest(), "-shared",
           *SOURCES, "-o", LIB]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError("building libxad_instruments.so failed:\n" + proc.stderr)
    return LIB


if __name__ == "__main__":
    print(build())
