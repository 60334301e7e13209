"""Host-side checks of device code whose arithmetic also runs on the CPU: the direct-to-LDS operand loaders
(tests/host_checks/loader_bounds.hip, built by the library's Makefile without any GPU code).  Every large-tile core
addresses its operands through these loaders, the register-staged core with plain buffer loads: every load of every
slab must stay inside the operand's window, and the window must be covered exactly once, for ragged limits and
contraction tails at the benchmark shapes' pitches."""

import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "gpu_ragged_dot_amd", "csrc")
EXE = os.path.join(ROOT, "tests", "host_checks", "loader_bounds")


def test_operand_loaders_stay_inside_their_windows():
    # (re)built on demand: a host-only compile of one file
    r = subprocess.run(["make", "-C", CSRC, os.path.relpath(EXE, CSRC)], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stdout + r.stderr
    r = subprocess.run([EXE], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stdout + r.stderr
    assert r.stdout.startswith("loader_bounds ok ") and int(r.stdout.split()[2]) > 10_000_000
