"""The host-side split-K geometry of the streaming matvec over the checkpoint layout, checked over a
sweep of shapes by a small C++ program built against the library (no GPU needed: plain host
arithmetic).  The case that matters: rows longer than 65280 positions in a layer small enough for
64-position units would need 256 or more workgroups per column tile, which the 8-bit arrival counter
of the accumulator word cannot count."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "mixed-precision-cuda-kernel_amd")
LIB = os.path.join(PKG, "libcherryq.so")


@pytest.mark.skipif(shutil.which("g++") is None or not os.path.isdir("/opt/rocm/include"),
                    reason="needs g++ and the HIP headers")
def test_matvec_geometry_keeps_splits_within_the_arrival_counter(tmp_path):
    assert os.path.exists(LIB), "build the library first (python mixed-precision-cuda-kernel_amd/build.py)"
    exe = str(tmp_path / "matvec_plan_check")
    cmd = ["g++", "-std=c++17", "-O1", "-D__HIP_PLATFORM_AMD__", "-I/opt/rocm/include",
           os.path.join(ROOT, "tests", "matvec_plan_check.cpp"), LIB, "-o", exe,
           f"-Wl,-rpath,{PKG}", "-Wl,-rpath,/opt/rocm/lib", "-L/opt/rocm/lib", "-lamdhip64"]
    subprocess.run(cmd, check=True, capture_output=True, text=True)
    run = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert run.returncode == 0, run.stdout[-2000:] + run.stderr[-2000:]
    assert " 0 bad" in run.stdout
