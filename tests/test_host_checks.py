"""Host-side checks of device code whose arithmetic also runs on the CPU: the direct-to-LDS operand loaders
(tests/host_checks/loader_bounds.hip, built by the library's Makefile without any GPU code).  Every large-tile core
addresses its operands through these loaders, the register-staged core with plain buffer loads: every load of every
slab must stay inside the operand's window, and the window must be covered exactly once, for ragged limits and
contraction tails at the benchmark shapes' pitches.  Likewise the rule that deals the blocks of long groups among those
of short groups in a gmm launch (tests/host_checks/block_order.hip): every block dealt once, evenly over the XCDs and
over the launch."""

import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "gpu_ragged_dot_amd", "csrc")
EXE = os.path.join(ROOT, "tests", "host_checks", "loader_bounds")
ORDER_EXE = os.path.join(ROOT, "tests", "host_checks", "block_order")


def test_operand_loaders_stay_inside_their_windows():
    # (re)built on demand: a host-only compile of one file
    r = subprocess.run(["make", "-C", CSRC, os.path.relpath(EXE, CSRC)], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stdout + r.stderr
    r = subprocess.run([EXE], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stdout + r.stderr
    assert r.stdout.startswith("loader_bounds ok ") and int(r.stdout.split()[2]) > 10_000_000


def test_interleaved_block_order_deals_every_block_once_and_evenly():
    r = subprocess.run(["make", "-C", CSRC, os.path.relpath(ORDER_EXE, CSRC)], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stdout + r.stderr
    r = subprocess.run([ORDER_EXE], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stdout + r.stderr
    assert r.stdout.startswith("block_order ok ") and int(r.stdout.split()[2]) > 1_000_000
