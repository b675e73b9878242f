"""Graphs of user kernels stay in vector registers on gfx950.

Compiles kernels written in the shapes users write (tests/native/resident/user_kernels.hip, and the
device example of the integration guide) at -O3 with the flags the guide prescribes, and once more
without the packed-fp32 switch (the instruction selection differs, and so did the outcome once), and
reads the code generator's own resource report: no scratch, no LDS (none of these kernels asks for
any: LDS here means that node state which the optimiser could not split was parked there), and a
ceiling on the vector registers of every kernel.

What this replaces in xyz-autodiff-cuda: `task ptx` / `task ptx-all` of Taskfile.yaml:27-147, which
emit the PTX of its caller, examples/mini-gaussian-splatting/gaussian_splatting_kernel.cu:73-111,
for inspection by hand.
"""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
KERNELS = os.path.join(ROOT, "tests", "native", "resident", "user_kernels.hip")

GUIDE_FLAGS = ["-munsafe-fp-atomics", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
FLAG_SETS = {"guide": GUIDE_FLAGS, "no_packed_switch": ["-munsafe-fp-atomics"]}

# vector-register ceilings: the figures of the day plus a few registers of slack for compiler noise
# (the two flag sets trade 40 against 42 on the broadcast graph)
VGPR_CEILING = {
    "resident_forward_loop": 36,
    "resident_run_loop": 40,
    "resident_broadcast_l1_run": 44,
    "resident_two_roots": 28,
    "resident_ternary": 16,
    "resident_repeated_forward": 16,
    "k": 24,  # the example of the integration guide
}


def _hipcc():
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("hipcc is not installed")
    return hipcc


def resource_report(source, flags, out_dir):
    """{kernel: {"vgprs", "scratch", "lds", "occupancy"}} from -Rpass-analysis=kernel-resource-usage."""
    cmd = [_hipcc(), "--offload-arch=gfx950", "-std=c++20", "-O3", "-I" + os.path.join(ROOT, "include"), *flags,
           "--cuda-device-only", "-c", str(source), "-o", os.path.join(str(out_dir), "resident.o"),
           "-Rpass-analysis=kernel-resource-usage"]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    assert proc.returncode == 0, proc.stderr
    report, name = {}, None
    fields = {"VGPRs": "vgprs", "ScratchSize [bytes/lane]": "scratch", "LDS Size [bytes/block]": "lds",
              "Occupancy [waves/SIMD]": "occupancy"}
    for line in proc.stderr.splitlines():
        m = re.search(r"remark:\s+Function Name: (\S+)", line)
        if m:
            name = m.group(1)
            mangled = re.match(r"_Z(\d+)(.*)", name)  # the guide's kernel is not extern "C": _Z1kPfS_ff
            if mangled:
                name = mangled.group(2)[: int(mangled.group(1))]
            report[name] = {}
            continue
        m = re.search(r"remark:\s+([A-Za-z][^:]*): (\d+)", line)
        if m and name and m.group(1).strip() in fields:
            report[name][fields[m.group(1).strip()]] = int(m.group(2))
    return report


def _check(report, names):
    assert set(names) <= set(report), (sorted(names), sorted(report))
    for name in names:
        r = report[name]
        assert r["scratch"] == 0, "%s spills: %d bytes of scratch per lane" % (name, r["scratch"])
        assert r["lds"] == 0, "%s: %d bytes of LDS per block hold node state that should be in registers" % (name, r["lds"])
        assert r["vgprs"] <= VGPR_CEILING[name], "%s: %d vector registers (ceiling %d)" % (name, r["vgprs"], VGPR_CEILING[name])
        assert r["occupancy"] == 8, (name, r)


@pytest.mark.parametrize("flag_set", sorted(FLAG_SETS))
def test_user_shaped_kernels_stay_in_registers(tmp_path, flag_set):
    report = resource_report(KERNELS, FLAG_SETS[flag_set], tmp_path)
    _check(report, [k for k in VGPR_CEILING if k != "k"])


def test_integration_example_stays_in_registers(tmp_path):
    text = open(os.path.join(ROOT, "INTEGRATION.md")).read()
    block = re.search(r"```cpp\n(#include <xyz_autodiff/xyz_autodiff\.cuh>.*?)```", text, re.S)
    assert block, "the example kernel is missing from the integration guide"
    src = tmp_path / "example.hip"
    src.write_text(block.group(1))
    report = resource_report(src, GUIDE_FLAGS, tmp_path)
    _check(report, ["k"])
