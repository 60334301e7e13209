"""The C ABI driven from a plain C program (tests/c_abi/abi_example.c, built by the library's Makefile with gcc):
no Python, no torch on that path.  The program checks the scheduling map bit for bit and both products against
host-side loops, and exits non-zero on any difference."""

import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
EXE = os.path.join(HERE, "c_abi", "abi_example")


def test_c_example_is_built():
    assert os.path.isfile(EXE) and os.access(EXE, os.X_OK), f"{EXE} missing: make -C gpu_ragged_dot_amd/csrc"


@pytest.mark.gpu
def test_c_example_runs_clean():
    print("plain C example", flush=True)
    r = subprocess.run([EXE], capture_output=True, text=True, timeout=100)
    print(r.stdout, r.stderr, flush=True)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "abi_example ok" in r.stdout
