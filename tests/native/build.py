"""Builds tests/native/libxad_api_tier.so (the API test tier) for gfx950 + host."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
LIB = os.path.join(HERE, "libxad_api_tier.so")


def build():
    cmd = [
        os.environ.get("HIPCC", "/opt/rocm/bin/hipcc"), "--offload-arch=gfx950", "-std=c++20", "-O2", "-fPIC", "-shared",
        "-fno-gpu-sanitize", "-march=x86-64-v3", "-munsafe-fp-atomics",
        "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument",
        "-I" + os.path.join(ROOT, "include"), "-I" + os.path.join(ROOT, "include", "mini-gaussian-splatting"),
        os.path.join(HERE, "api_tier.hip"), "-o", LIB,
    ]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        noise = "is not a recognized feature for this target"
        raise RuntimeError("hipcc failed:\n" + "\n".join(l for l in proc.stderr.splitlines() if noise not in l))
    return LIB


if __name__ == "__main__":
    print(build())
