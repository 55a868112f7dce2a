"""Runs tests/tuning_variants.py (every tile walk, cache policy and window form of the transposing kernel, forced in
turn) in a child process whose environment switches the library's tuning aids on: MONARCH_HIP_TUNING=1 must be set when
the library is loaded, and this process has loaded it without."""
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.gpu
@pytest.mark.timeout(600)
def test_forced_variants_of_the_transposing_kernel_move_the_same_bytes():
    env = dict(os.environ, MONARCH_HIP_TUNING="1")
    r = subprocess.run([sys.executable, "-u", "-m", "pytest", "-x", "-q", "-m", "gpu", "--timeout", "300", "--timeout-method", "thread",
                        "-p", "no:cacheprovider", "tests/tuning_variants.py"], cwd=ROOT, env=env, capture_output=True, text=True,
                       timeout=550)
    assert r.returncode == 0, r.stdout[-4000:] + r.stderr[-2000:]
    assert " passed" in r.stdout and "skipped" not in r.stdout
