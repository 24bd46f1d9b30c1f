"""The launch sizes of the compacted backward against its device-made work plan, on the host (no GPU): the library's own
split and bound functions (flash-dmattn_amd/csrc/fdma_params.h) are compiled into tests/host/plan_bounds_check.cpp with
g++ and swept over pair counts, group sizes and ragged unit counts.  A per-XCD list of the plan that held more parts
than the launch has workgroups for would leave parts out of the dK / dV sums (the plan flags it and the gradients turn
into NaN): the sweep shows that the host-side bound covers every plan the device can make."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.skipif(shutil.which("g++") is None, reason="no host compiler")
def test_host_bounds_cover_every_plan(tmp_path):
    exe = str(tmp_path / "plan_bounds_check")
    cmd = ["g++", "-O1", "-std=c++17", "-D__HIP_PLATFORM_AMD__", "-I/opt/rocm/include",
           "-I" + os.path.join(ROOT, "flash-dmattn_amd", "csrc"), os.path.join(ROOT, "tests", "host", "plan_bounds_check.cpp"), "-o", exe]
    build = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert build.returncode == 0, build.stderr[-2000:]
    run = subprocess.run([exe], capture_output=True, text=True, timeout=300)
    assert run.returncode == 0 and run.stdout.strip().splitlines()[-1].startswith("OK"), run.stdout[-2000:]
