"""Builds tests/native/libxad_api_tier.so (the API test tier, hipcc: gfx950 + host pass) and
tests/native/libxad_tester_host.so (the gradient testers compiled by g++ alone)."""
import hashlib
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
LIB = os.path.join(HERE, "libxad_api_tier.so")
HOST_LIB = os.path.join(HERE, "libxad_tester_host.so")


def source_digest():
    """SHA-256 over this directory's sources and the library headers they include."""
    h = hashlib.sha256()
    files = [os.path.join(HERE, f) for f in os.listdir(HERE) if f.endswith((".hip", ".cuh", ".inc", ".cpp"))]
    for dirpath, _, names in os.walk(os.path.join(ROOT, "include")):
        files += [os.path.join(dirpath, f) for f in names if f.endswith((".cuh", ".h"))]
    # the compositing kernels' visibility test, which the tier runs on both sides
    files += [os.path.join(ROOT, "xyz_autodiff_cuda_amd", "csrc", f) for f in ("splat_staged.cuh", "splat.cuh")]
    for path in sorted(files):
        h.update(os.path.relpath(path, ROOT).encode() + b"\0")
        with open(path, "rb") as f:
            h.update(f.read() + b"\0")
    return h.hexdigest()


def build():
    cmd = [
        os.environ.get("HIPCC", "/opt/rocm/bin/hipcc"), "--offload-arch=gfx950", "-std=c++20", "-O2", "-fPIC", "-shared",
        "-fno-gpu-sanitize", "-march=x86-64-v3", "-munsafe-fp-atomics",
        "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument",
        "-I" + os.path.join(ROOT, "include"), "-I" + os.path.join(ROOT, "include", "mini-gaussian-splatting"),
        "-DXAD_TEST_SOURCE_DIGEST=\"%s\"" % source_digest(),
        os.path.join(HERE, "api_tier.hip"), "-o", LIB,
    ]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        noise = "is not a recognized feature for this target"
        raise RuntimeError("hipcc failed:\n" + "\n".join(l for l in proc.stderr.splitlines() if noise not in l))
    host = [
        os.environ.get("CXX", "g++"), "-std=c++20", "-O1", "-fPIC", "-shared", "-march=x86-64-v3",
        "-I" + os.path.join(ROOT, "include"), "-I" + os.path.join(ROOT, "include", "mini-gaussian-splatting"),
        "-DXAD_TEST_SOURCE_DIGEST=\"%s\"" % source_digest(),
        os.path.join(HERE, "tester_host.cpp"), "-o", HOST_LIB,
    ]
    proc = subprocess.run(host, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError("g++ failed:\n" + proc.stderr)
    return LIB


if __name__ == "__main__":
    print(build())
