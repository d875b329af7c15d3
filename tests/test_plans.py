"""The launch plans of the kernels (csrc/plans.h: K slices, grids, LDS bytes, workspace offsets) are host code; here
they are compiled for the CPU with the address and undefined-behaviour sanitizers and swept over shapes
(tests/plans_check.cpp).  The reference runs sanitizers over the host code that parses untrusted input
(.github/workflows/fuzz.yml:34); the counterpart here is the code whose mistakes would be device faults."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_launch_plans_hold_under_the_sanitizers(tmp_path):
    compiler = shutil.which("g++") or shutil.which("clang++")
    if compiler is None:
        pytest.skip("no host C++ compiler")
    binary = str(tmp_path / "plans_check")
    build = subprocess.run([compiler, "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=all",
                            "-I", os.path.join(ROOT, "fllm_amd", "csrc"), os.path.join(ROOT, "tests", "plans_check.cpp"), "-o", binary],
                           capture_output=True, text=True, timeout=300)
    assert build.returncode == 0, build.stderr
    run = subprocess.run([binary], capture_output=True, text=True, timeout=120,
                         env=dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0"))
    assert run.returncode == 0, run.stdout + run.stderr
    assert "plans ok" in run.stdout
