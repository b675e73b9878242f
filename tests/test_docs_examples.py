"""The device-code example of INTEGRATION.md is compiled as it stands in the document."""
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
    assert block, "the example kernel is missing from INTEGRATION.md"
    src = tmp_path / "example.hip"
    src.write_text(block.group(1))
    cmd = [hipcc, "--offload-arch=gfx950", "-std=c++20", "-O1", "-I" + os.path.join(ROOT, "include"), "-munsafe-fp-atomics",
           "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "--cuda-device-only", "-c", str(src), "-o",
           str(tmp_path / "example.o")]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    assert proc.returncode == 0, proc.stderr
