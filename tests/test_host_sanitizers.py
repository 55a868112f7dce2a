"""The library's host code (Slice semantics in slice_host.cpp, copy planning in plan.cpp, work-queue and
completion-queue entries built on the calling thread in rdmaxcel_host.cpp) is plain C++:
it is compiled here with the host compiler under AddressSanitizer and UndefinedBehaviorSanitizer together
with tests/c_abi/host_fuzz.cpp, which drives thousands of random valid and invalid Slices and queue parameters through
every host entry point and compares the results with the definitions."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_host_code_under_address_and_ub_sanitizers(tmp_path):
    if shutil.which("g++") is None:
        pytest.skip("no host C++ compiler")
    exe = str(tmp_path / "host_fuzz")
    csrc = os.path.join(ROOT, "monarch_amd", "csrc")
    build = subprocess.run(["g++", "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=all",
                            "-Wall", "-Wextra", os.path.join(ROOT, "tests", "c_abi", "host_fuzz.cpp"),
                            os.path.join(csrc, "slice_host.cpp"), os.path.join(csrc, "plan.cpp"), os.path.join(csrc, "rdmaxcel_host.cpp"),
                            "-o", exe],
                           capture_output=True, text=True)
    if build.returncode != 0 and "sanitizer" in build.stderr.lower() and "cannot find" in build.stderr.lower():
        pytest.skip("sanitizer runtimes are not installed")
    assert build.returncode == 0 and not build.stderr.strip(), build.stderr[-3000:]  # -Wall -Wextra clean, too
    run = subprocess.run([exe], capture_output=True, text=True, timeout=300)
    assert run.returncode == 0 and run.stdout.startswith("ok:"), (run.stdout[-2000:], run.stderr[-3000:])
