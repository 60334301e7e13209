"""Seeded random cases against the oracle: shapes (aligned and odd pitches, a few with several rounds of 256 x 256
tiles or a long contraction), group sizes (random partitions, Zipf-like with empty groups, everything in one group,
lengths around tile boundaries, all empty; with and without a zero tail), bf16, float32 and float16, all three products, the
default plan or a random compiled variant with a random tile walk and K-split setting, and the streaming kernels forced.
A call the library refuses must refuse with RD_ERR_UNSUPPORTED or RD_ERR_INVALID_ARGUMENT; everything it accepts must
match the oracle at the reference's tolerances (tests.py:127,144,168,183; float32 5e-4 / 1e-4, tests.py:93; float16 a
fifth / half of the bf16 ones), with the
tail rows and the empty groups' slices exactly zero."""

import numpy as np
import pytest
import torch

from gpu_ragged_dot_amd import _capi, ops
from oracle import ragged_dot_oracle as oracle
from tests import util

pytestmark = pytest.mark.gpu

HP = dict(block_m=64, block_k=64, block_n=64, interpret=False, compute_dtype=None, acc_dtype=torch.float32, chunk_m=512)


def _dim(rng, lo, hi, aligned):
    v = int(rng.integers(lo, hi + 1))
    return max(8, (v + 7) // 8 * 8) if aligned else v


def _group_sizes(rng, g, m):
    kind = int(rng.integers(0, 5))
    target = m if rng.random() < 0.5 else int(rng.integers(0, m + 1))
    if kind == 0:    # a random partition
        cuts = np.sort(rng.integers(0, target + 1, size=g - 1)) if g > 1 else np.array([], int)
        gs = np.diff(np.concatenate([[0], cuts, [target]]))
    elif kind == 1:  # Zipf-like, some groups empty
        p = (rng.permutation(g) + 1.0) ** -1.2
        p[rng.random(g) < 0.3] = 0
        if p.sum() == 0:
            p[0] = 1
        gs = rng.multinomial(target, p / p.sum())
    elif kind == 2:  # everything in one group
        gs = np.zeros(g, int)
        gs[rng.integers(0, g)] = target
    elif kind == 3:  # lengths around tile boundaries
        gs = rng.choice(np.array([0, 1, 31, 32, 33, 63, 64, 65, 127, 128, 129, 255, 256, 257]), size=g)
        while gs.sum() > target and gs.sum() > 0:
            gs[rng.integers(0, g)] //= 2
    else:            # all empty
        gs = np.zeros(g, int)
    return gs.astype(np.int32)


def _one_case(seed, it, variants):
    rng = np.random.default_rng(seed * 100003 + it)
    op = ["gmm", "gmm_t", "tgmm"][int(rng.integers(0, 3))]
    dt = ["bfloat16", "float32", "float16"][int(np.searchsorted([0.7, 0.85], rng.random(), side="right"))]
    aligned = rng.random() < 0.7
    big = rng.random() < 0.25
    m = int(rng.integers(1, 2500 if big else 600))
    k = _dim(rng, 1, 1300 if big else 300, aligned)   # contraction length of gmm; rows of the tgmm result
    n = _dim(rng, 1, 1300 if big else 300, aligned)
    g = int(rng.integers(1, 40))
    cat = rng.random()
    if cat < 0.12 and op != "tgmm":   # several rounds of 256 x 256 tiles over a short contraction
        m = int(rng.integers(2000, 9000))
        n = int(rng.integers(8, 19)) * 256 + (0 if rng.random() < 0.5 else 8 * int(rng.integers(0, 31)))
        k = _dim(rng, 16, 160, True)
        aligned, g = True, int(rng.integers(1, 70))
    elif cat < 0.22:                  # a long contraction (tgmm: tall result slices)
        m = int(rng.integers(256, 1500))
        n, k, aligned = _dim(rng, 256, 1024, True), _dim(rng, 1024, 9000, True), True
        g = int(rng.integers(1, 12))
    if op == "tgmm" and g * k * n > 3e7:
        g = max(1, int(3e7 // (k * n)))
    gs = _group_sizes(rng, g, m)
    plan, plan_txt = None, "default"
    if rng.random() < 0.6:
        code = {"bfloat16": _capi.RD_DTYPE_BF16, "float32": _capi.RD_DTYPE_F32, "float16": _capi.RD_DTYPE_F16}[dt]
        cand = [v for v in variants if v.dtype == code and (not v.vec or aligned)]
        v = cand[int(rng.integers(0, len(cand)))]
        gm, gn, sk = int(rng.integers(0, 9)), int(rng.integers(0, 9)), int(rng.choice([0, 0, -1, 2, 8]))
        plan, plan_txt = _capi.Plan(v.id, gm, 0, gn, sk), f"{v.name.decode()}:{gm}:{gn}:split_k={sk}"
    elif rng.random() < 0.3 and op != "tgmm":
        plan = _capi.Plan(-1, 0, int(rng.choice([-1, 32, 64, 128])), 0, 0)
        plan_txt = f"decode_nb={plan.decode_nb}"
    what = f"case {seed}/{it}: {op} {dt} m={m} k={k} n={n} g={g} sum={int(gs.sum())} max={int(gs.max())} plan={plan_txt}"
    print(what, flush=True)
    x = oracle.round_to(rng.standard_normal((m, k)).astype(np.float32), dt)
    w = oracle.round_to((rng.standard_normal((g, k, n)) / max(k, 1) ** 0.5).astype(np.float32), dt)
    d = oracle.round_to(rng.standard_normal((m, n)).astype(np.float32), dt)
    tdt = {"bfloat16": torch.bfloat16, "float32": torch.float32, "float16": torch.float16}[dt]
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda().to(tdt)
    eps_rows = {"bfloat16": util.BF16_EPS, "float32": 5e-4, "float16": util.BF16_EPS / 5}[dt]
    eps_groups = {"bfloat16": util.TGMM_BF16_EPS, "float32": 1e-4, "float16": util.TGMM_BF16_EPS / 2}[dt]
    live = int(gs.sum())
    try:
        if op == "gmm":
            got = util.to_np(ops._gmm_fwd(dev(x), dev(w), torch.from_numpy(gs), **HP, trans_rhs=False, plan=plan))
            util.assert_close_rows(got, oracle.gmm(x, w, gs, out_dtype=dt), live, eps_rows, what)
            assert not np.any(got[live:]), what
        elif op == "gmm_t":   # the weights [g, k, n] read as [g, n', k'] with n' = k: y = d . w[g]^T, contraction over n
            got = util.to_np(ops._gmm_fwd(dev(d), dev(w), torch.from_numpy(gs), **HP, trans_rhs=True, plan=plan))
            util.assert_close_rows(got, oracle.gmm(d, w, gs, trans_rhs=True, out_dtype=dt), live, eps_rows, what)
            assert not np.any(got[live:]), what
        else:
            got = util.to_np(ops._tgmm_fwd(dev(x), dev(d), torch.from_numpy(gs), **HP, plan=plan))
            if np.any(gs != 0):
                util.assert_close_groups(got, oracle.tgmm(x, d, gs, out_dtype=dt), gs != 0, eps_groups, what)
            assert not np.any(got[gs == 0]), what
    except _capi.RaggedDotError as e:
        assert e.status in (_capi.RD_ERR_UNSUPPORTED, _capi.RD_ERR_INVALID_ARGUMENT), f"{what}: {e}"
        return False
    return True


@pytest.mark.parametrize("seed", [11, 12, 13])
def test_random_cases_against_the_oracle(seed):
    variants = _capi.variants()
    ran = sum(_one_case(seed, it, variants) for it in range(150))
    assert ran >= 120   # refusals (a streaming kernel forced on a shape it does not serve) stay the exception
