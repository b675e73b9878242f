"""Builds libxad_hip.so (HIP kernels + C ABI) for gfx950, in-tree.

    python -m xyz_autodiff_cuda_amd.build

hipcc cross-compiles without a GPU.  The host pass of the same translation
units carries the host-core build of the templates (x86-64-v3: AVX2 + FMA, so
the library runs on any recent host without depending on the build machine).
"""
import hashlib
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
TRAINER = os.path.join(CSRC, "trainer")
LIB = os.path.join(HERE, "libxad_hip.so")
TRAIN_BIN = os.path.join(HERE, "xad_splat_train")
OBJ_DIR = os.path.join(HERE, "build")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

FLAGS = [
    "--offload-arch=gfx950",
    "-std=c++20",
    "-O3",
    "-fPIC",
    "-fno-gpu-sanitize",
    "-march=x86-64-v3",
    "-munsafe-fp-atomics",
    # x + 0 folds away (gradients start from zero); fp32 division is v_rcp_f32
    # based (2.5 ulp) instead of the IEEE sequence
    "-fno-signed-zeros",
    "-fno-hip-fp32-correctly-rounded-divide-sqrt",
    # keep v_pk_*_f32 out of the generated code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    "-I" + os.path.join(ROOT, "include"),
    "-I" + os.path.join(ROOT, "include", "mini-gaussian-splatting"),
]


def sources():
    """Translation units of the library: the kernels and, under trainer/, the host-only front-end."""
    units = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip")]
    units += [os.path.join(TRAINER, f) for f in os.listdir(TRAINER) if f.endswith((".hip", ".cpp")) and f != "train_main.cpp"]
    return sorted(units)


def source_digest():
    """SHA-256 over every file the library is built from (csrc/ and include/), by
    relative path and content.  The build bakes it into the library
    (xad_source_digest) so that a library older than its sources can be told."""
    h = hashlib.sha256()
    files = []
    for base in (CSRC, os.path.join(ROOT, "include")):
        for dirpath, _, names in os.walk(base):
            files += [os.path.join(dirpath, f) for f in names if f.endswith((".hip", ".cuh", ".h", ".cpp"))]
    for path in sorted(files):
        h.update(os.path.relpath(path, ROOT).encode())
        h.update(b"\0")
        with open(path, "rb") as f:
            h.update(f.read())
        h.update(b"\0")
    return h.hexdigest()


def _compile(src, digest):
    obj = os.path.join(OBJ_DIR, os.path.relpath(src, CSRC).replace(os.sep, "_") + ".o")
    cmd = [HIPCC, *FLAGS, "-DXAD_SOURCE_DIGEST=\"%s\"" % digest, "-c", src, "-o", obj]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in proc.stderr.splitlines() if noise not in l)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, err))
    return obj, err


def build(verbose=False):
    os.makedirs(OBJ_DIR, exist_ok=True)
    digest = source_digest()
    with ThreadPoolExecutor(max_workers=min(8, os.cpu_count() or 1)) as pool:
        results = list(pool.map(lambda src: _compile(src, digest), sources()))
    objs = [o for o, _ in results]
    if verbose:
        for _, err in results:
            if err.strip():
                print(err, file=sys.stderr)
    link = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-sanitize", "-o", LIB, *objs, "-lpthread", "-lz"]
    proc = subprocess.run(link, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError("link failed:\n" + proc.stderr)
    # the trainer program: plain C++ on the C ABI, finds the library next to itself
    program = ["g++", "-std=c++17", "-O2", "-Wall", "-Wextra", os.path.join(TRAINER, "train_main.cpp"), "-o", TRAIN_BIN,
               "-L" + HERE, "-lxad_hip", "-Wl,-rpath,$ORIGIN", "-Wl,-rpath-link," + os.path.join(os.path.dirname(os.path.dirname(HIPCC)), "lib")]
    proc = subprocess.run(program, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError("building xad_splat_train failed:\n" + proc.stderr)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
