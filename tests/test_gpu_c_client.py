"""The C ABI driven from plain C: tests/c_abi/c_client.c allocates device memory, uploads data and
times a launch through the runtime pass-through symbols, runs pack/unpack, the bf16 reduce and the fp8
codec, and checks the results against loops of its own.  No Python, torch or oracle in that process."""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
SRC = os.path.join(HERE, "c_abi", "c_client.c")
BIN = os.path.join(HERE, "c_abi", "c_client")


def build_c_client(out: str = BIN) -> str:
    subprocess.check_call(["gcc", "-std=c11", "-O1", "-Wall", "-Wextra", "-Werror", "-I", os.path.join(ROOT, "include"), SRC,
                           "-o", out, "-L", os.path.join(ROOT, "monarch_amd"), "-lmonarch_hip",
                           "-Wl,-rpath," + os.path.join(ROOT, "monarch_amd"), "-lm"])
    return out


def test_c_client_compiles_and_links(tmp_path):
    # host only: the header is enough for a C compiler and every symbol the client uses resolves
    build_c_client(str(tmp_path / "c_client"))


@pytest.mark.gpu
def test_c_client_runs():
    if not os.path.exists(BIN) or os.path.getmtime(BIN) < os.path.getmtime(SRC):
        build_c_client()
    res = subprocess.run([BIN], capture_output=True, text=True, timeout=120)
    assert res.returncode == 0, res.stdout + res.stderr
    assert "c_client ok" in res.stdout
