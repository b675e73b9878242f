"""The device-code example of the integration guide is compiled as it stands in the document."""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_integration_example_compiles_for_gfx950(tmp_path):
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("hipcc is not installed")
    text = open(os.path.join(ROOT, "INTEGRATION.md")).read()
    block = re.search(r"```cpp\n(#include <xyz_autodiff/xyz_autodiff\.cuh>.*?)```", text, re.S)
    assert block, "the example kernel is missing from the integration guide"
    src = tmp_path / "example.hip"
    src.write_text(block.group(1))
    cmd = [hipcc, "--offload-arch=gfx950", "-std=c++20", "-O1", "-I" + os.path.join(ROOT, "include"), "-munsafe-fp-atomics",
           "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "--cuda-device-only", "-c", str(src), "-o",
           str(tmp_path / "example.o")]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    assert proc.returncode == 0, proc.stderr


def test_integration_host_stub_compiles(tmp_path):
    """The C++ stubs of the integration guide against include/xad_capi.h (syntax and types only)."""
    gxx = shutil.which("g++")
    hip_include = "/opt/rocm/include"
    if not gxx or not os.path.exists(os.path.join(hip_include, "hip", "hip_runtime_api.h")):
        pytest.skip("g++ or the HIP headers are not installed")
    text = open(os.path.join(ROOT, "INTEGRATION.md")).read()
    block = re.search(r"```cpp\n(// replaces launch_gaussian_splatting.*?)```", text, re.S)
    assert block, "the host stub is missing from the integration guide"
    prelude = ("#include <cstddef>\n#include <stdexcept>\n#include <hip/hip_runtime_api.h>\n"
               "static float lr_pos = 1e-2f, lr_scale = 1e-2f, lr_rot = 1e-2f, lr_col = 1e-2f, lr_opacity = 1e-2f;\n")
    src = tmp_path / "stub.cpp"
    src.write_text(prelude + block.group(1))
    cmd = [gxx, "-std=c++17", "-fsyntax-only", "-D__HIP_PLATFORM_AMD__", "-I" + hip_include, "-I" + os.path.join(ROOT, "include"), str(src)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    assert proc.returncode == 0, proc.stderr
