"""Shared helpers for the parity tests: seeded inputs in the style of the reference's tests.py and conversions
between torch bf16 device tensors and the float32 numpy arrays the oracle works on."""

import itertools
import random

import numpy as np
import torch

from oracle import ragged_dot_oracle as oracle

BF16_EPS = 5e-3  # tests.py:127,144,168
TGMM_BF16_EPS = 2e-3  # tests.py:183
NORTH_STAR_TOL = 1e-2  # max|diff| <= 1e-2 * max|ref|


def to_np(t: torch.Tensor) -> np.ndarray:
    return t.detach().float().cpu().numpy()


def bf16_dev(a: np.ndarray, device="cuda") -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(device).to(torch.bfloat16)


def make_case(seed, m, k, n, g, fill_in, random_inputs, scale_rhs=False):
    """Inputs like tests.py:51-71,109-117: N(0,1) (or all-ones) rounded to bf16, softmax-distributed group sizes."""
    rng = np.random.default_rng(seed * 7919 + m * 31 + k * 17 + n * 13 + g)
    if random_inputs:
        lhs = rng.normal(size=(m, k)).astype(np.float32)
        rhs = rng.normal(size=(g, k, n)).astype(np.float32)
        dout = rng.normal(size=(m, n)).astype(np.float32)
        if scale_rhs:
            rhs /= np.sqrt(k)
    else:
        lhs, rhs, dout = (np.ones(s, dtype=np.float32) for s in ((m, k), (g, k, n), (m, n)))
    lhs, rhs, dout = (oracle.round_to(a, "bfloat16") for a in (lhs, rhs, dout))
    target_m = max(min(round(m * fill_in), m), 0)
    gs = oracle.generate_group_sizes(seed + 1000 * g + target_m, g, target_m)
    return lhs, rhs, dout, gs, target_m


def reference_grid(samples: int, seed: int = 0):
    """A seeded sample of the reference's parameter grid (tests.py:91-105), bf16 cases."""
    grid = dict(
        m=[128, 256, 171],
        k=[256, 512, 58],
        n=[64, 128, 77],
        g=[8, 16],
        block_m=[16, 32, 64],
        block_k=[16, 32, 64],
        block_n=[16, 32, 64],
        fill_in=[1.0, 0.7, 0.5],
        seed=[0, 1],
        random_inputs=[True, False],
        chunk_m=[8, 512],
    )
    keys = list(grid)
    combos = list(itertools.product(*grid.values()))
    random.Random(seed).shuffle(combos)
    return [dict(zip(keys, c)) for c in combos[:samples]]


def case_id(c: dict) -> str:
    return "-".join(f"{k[0]}{k[-1]}{v}" for k, v in c.items())


def assert_close_rows(got, ref, target_m, eps, what):
    err = oracle.err_fn(got, ref, axis=-1, mask=np.arange(ref.shape[0]) < target_m)
    assert float(np.max(err)) < eps, f"{what}: max row rel-L2 {np.max(err):.3e} >= {eps}"
    tol = NORTH_STAR_TOL * max(float(np.max(np.abs(ref))), 1e-30)
    assert float(np.max(np.abs(got - ref))) <= tol, f"{what}: max|diff| {np.max(np.abs(got - ref)):.3e} > {tol:.3e}"


def assert_close_groups(got, ref, mask, eps, what):
    err = oracle.err_fn(got, ref, axis=(-1, -2), mask=mask)
    assert float(np.max(err)) < eps, f"{what}: max group rel-Frobenius {np.max(err):.3e} >= {eps}"
    tol = NORTH_STAR_TOL * max(float(np.max(np.abs(ref))), 1e-30)
    assert float(np.max(np.abs(got - ref))) <= tol, f"{what}: max|diff| {np.max(np.abs(got - ref)):.3e} > {tol:.3e}"
