"""Token routing around ragged_dot: the numpy oracle pinned on the CPU, the HIP kernels against it on the GPU.

The reference has no counterpart (its caller sorts the rows), so the oracle is pinned by brute force, invariants,
adjointness and a committed fixture rather than by reference vectors.
"""

import json
import os

import numpy as np
import pytest
import torch

from oracle import moe_glue_oracle as moe_oracle
from oracle import ragged_dot_oracle as oracle
from tests import util

HERE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
ROUTES = json.load(open(os.path.join(HERE, "moe_route_golden.json")))


def _brute_route(ids, g):
    """Append every kept slot, in slot order, to its expert's list; concatenate the lists."""
    flat = [int(v) for v in np.asarray(ids).reshape(-1)]
    lists = [[] for _ in range(g)]
    for s, e in enumerate(flat):
        if 0 <= e < g:
            lists[e].append(s)
    rows = [s for lst in lists for s in lst]
    ros = [-1] * len(flat)
    for r, s in enumerate(rows):
        ros[s] = r
    return [len(lst) for lst in lists], ros, rows + [-1] * (len(flat) - len(rows))


def _random_ids(seed, tokens, top_k, g, drop=0.0):
    rng = np.random.default_rng(seed)
    ids = rng.integers(0, g, size=(tokens, top_k)).astype(np.int32)
    if drop:
        ids[rng.random(ids.shape) < drop] = rng.choice([-1, g, g + 5])
    return ids


# ---------------------------------------------------------------------------------------------------------------------
# oracle on the CPU
# ---------------------------------------------------------------------------------------------------------------------

@pytest.mark.parametrize("seed,tokens,top_k,g,drop", [(0, 1, 1, 1, 0), (1, 7, 2, 3, 0), (2, 40, 3, 5, 0.2),
                                                       (3, 64, 8, 128, 0), (4, 33, 4, 2, 0.5), (5, 0, 2, 4, 0)])
def test_oracle_route_matches_brute_force(seed, tokens, top_k, g, drop):
    ids = _random_ids(seed, tokens, top_k, g, drop)
    gs, ros, sor = moe_oracle.route(ids, g)
    bgs, bros, bsor = _brute_route(ids, g)
    assert gs.tolist() == bgs and ros.tolist() == bros and sor.tolist() == bsor


def test_oracle_route_invariants():
    ids = _random_ids(11, 300, 4, 17, 0.1)
    gs, ros, sor = moe_oracle.route(ids, 17)
    flat = ids.reshape(-1)
    total = int(gs.sum())
    kept = (flat >= 0) & (flat < 17)
    assert total == kept.sum() and (ros >= 0).sum() == total and (sor >= 0).sum() == total
    assert np.array_equal(sor[ros[kept]], np.nonzero(kept)[0])          # inverse permutations
    experts_in_row_order = flat[sor[:total]]
    assert np.all(np.diff(experts_in_row_order) >= 0)                    # sorted by expert
    same = np.diff(experts_in_row_order) == 0
    assert np.all(np.diff(sor[:total])[same] > 0)                        # stable inside an expert
    assert np.array_equal(np.bincount(experts_in_row_order, minlength=17), gs)
    assert np.all(sor[total:] == -1) and np.all(ros[~kept] == -1)


@pytest.mark.parametrize("i", range(len(ROUTES)))
def test_oracle_reproduces_route_fixture(i):
    fx = ROUTES[i]
    gs, ros, sor = moe_oracle.route(np.array(fx["expert_ids"], np.int32), fx["g"])
    assert gs.tolist() == fx["group_sizes"] and ros.tolist() == fx["row_of_slot"] and sor.tolist() == fx["slot_of_row"]


def test_route_fixture_known_answer():
    fx = ROUTES[0]  # ids [[2,0],[1,2],[0,0],[3,1]], g=4: by hand
    assert fx["group_sizes"] == [3, 2, 2, 1]
    assert fx["slot_of_row"] == [1, 4, 5, 2, 7, 0, 3, 6]
    assert fx["row_of_slot"] == [5, 0, 3, 6, 1, 2, 7, 4]


def test_oracle_dispatch_combine_adjoint_and_definition():
    rng = np.random.default_rng(3)
    tokens, top_k, g, d = 29, 3, 7, 11
    ids = _random_ids(21, tokens, top_k, g, 0.15)
    _, ros, sor = moe_oracle.route(ids, g)
    h = rng.standard_normal((tokens, d)).astype(np.float32)
    y = rng.standard_normal((tokens * top_k, d)).astype(np.float32)
    w = rng.standard_normal((tokens, top_k)).astype(np.float32)
    x = moe_oracle.dispatch(h, sor, top_k)
    for r, s in enumerate(sor):                                          # definition, row by row
        assert np.array_equal(x[r], h[s // top_k] if s >= 0 else np.zeros(d, np.float32))
    lhs = np.sum(x.astype(np.float64) * y)
    rhs = np.sum(h.astype(np.float64) * moe_oracle.combine(y, ros, top_k))
    assert abs(lhs - rhs) <= 1e-9 * max(abs(lhs), 1)
    out = moe_oracle.combine(y, ros, top_k, w)
    t = 5
    want = sum(w[t, s] * y[ros[t * top_k + s]].astype(np.float64) for s in range(top_k) if ros[t * top_k + s] >= 0)
    assert np.allclose(out[t], want, rtol=1e-12, atol=1e-12)
    # adjoint of the weighted combine with respect to y is the scaled dispatch; with respect to w, combine_wgrad
    dout = rng.standard_normal((tokens, d)).astype(np.float32)
    dy = moe_oracle.dispatch(dout, sor, top_k, row_scale=w)
    assert abs(np.sum(out * dout) - np.sum(dy.astype(np.float64) * y)) <= 1e-5 * abs(np.sum(out * dout))
    dw = moe_oracle.combine_wgrad(y, dout, ros, top_k)
    eps = 1e-3
    w2 = w.copy(); w2[t, 1] += eps
    fd = (np.sum(moe_oracle.combine(y, ros, top_k, w2) * dout) - np.sum(out * dout)) / eps
    assert abs(fd - dw[t, 1]) <= 1e-4 * max(abs(fd), 1)


# ---------------------------------------------------------------------------------------------------------------------
# HIP kernels on the GPU
# ---------------------------------------------------------------------------------------------------------------------

ROUTE_CASES = [(0, 1, 1, 1, 0), (1, 7, 2, 3, 0), (2, 40, 3, 5, 0.2), (3, 8, 8, 128, 0), (4, 33, 4, 2, 0.5),
               (6, 4096, 8, 256, 0.0), (7, 5000, 2, 8, 0.05), (8, 3000, 6, 1500, 0.1), (9, 1030, 1, 12288, 0.0),
               (10, 250000, 2, 12288, 0.01),   # per-chunk histograms would pass 4M entries: the chunk length doubles
               (11, 2000, 64, 32, 0.0)]       # the largest top_k


@pytest.mark.gpu
@pytest.mark.parametrize("seed,tokens,top_k,g,drop", ROUTE_CASES, ids=[f"t{c[1]}k{c[2]}g{c[3]}" for c in ROUTE_CASES])
def test_route_bit_exact(seed, tokens, top_k, g, drop):
    from gpu_ragged_dot_amd import moe
    print(f"route tokens={tokens} top_k={top_k} g={g} drop={drop}", flush=True)
    ids = _random_ids(seed, tokens, top_k, g, drop)
    r = moe.route(torch.from_numpy(ids).cuda(), g)
    gs, ros, sor = moe_oracle.route(ids, g)
    assert np.array_equal(r.group_sizes.cpu().numpy(), gs)
    assert np.array_equal(r.row_of_slot.cpu().numpy(), ros)
    assert np.array_equal(r.slot_of_row.cpu().numpy(), sor)


@pytest.mark.gpu
@pytest.mark.parametrize("i", range(len(ROUTES)))
def test_route_fixture_on_gpu(i):
    from gpu_ragged_dot_amd import moe
    fx = ROUTES[i]
    r = moe.route(torch.tensor(fx["expert_ids"], dtype=torch.int32).cuda(), fx["g"])
    assert r.group_sizes.cpu().tolist() == fx["group_sizes"]
    assert r.row_of_slot.cpu().tolist() == fx["row_of_slot"] and r.slot_of_row.cpu().tolist() == fx["slot_of_row"]


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16], ids=["bf16", "f32", "f16"])
@pytest.mark.parametrize("tokens,top_k,g,d", [(64, 8, 128, 2048), (300, 2, 8, 520), (77, 3, 5, 58), (1000, 4, 16, 7)])
def test_dispatch_combine_parity(tokens, top_k, g, d, dtype):
    """dispatch is a copy: bit-exact.  combine sums top_k products in fp32 and rounds once: within 2^-7 (bf16), 2^-10
    (float16) or 1e-5 (float32) of the float64 oracle, relative to the largest output."""
    from gpu_ragged_dot_amd import moe
    print(f"dispatch/combine tokens={tokens} top_k={top_k} g={g} d={d} {dtype}", flush=True)
    rng = np.random.default_rng(tokens + d)
    ids = _random_ids(tokens, tokens, top_k, g, 0.1)
    name = {torch.bfloat16: "bfloat16", torch.float32: "float32", torch.float16: "float16"}[dtype]
    rnd = lambda a: oracle.round_to(a, name)
    h = rnd(rng.standard_normal((tokens, d)).astype(np.float32))
    y = rnd(rng.standard_normal((tokens * top_k, d)).astype(np.float32))
    w = rng.random((tokens, top_k)).astype(np.float32)
    r = moe.route(torch.from_numpy(ids).cuda(), g)
    _, ros, sor = moe_oracle.route(ids, g)
    hd, yd, wd = (torch.from_numpy(a).cuda() for a in (h, y, w))
    x = moe.dispatch(hd.to(dtype), r)
    assert np.array_equal(util.to_np(x), moe_oracle.dispatch(h, sor, top_k))
    tol = {torch.bfloat16: 2.0 ** -7, torch.float32: 1e-5, torch.float16: 2.0 ** -10}[dtype]
    for weights, wn in ((None, None), (wd, w)):
        out = util.to_np(moe.combine(yd.to(dtype), r, weights))
        ref = moe_oracle.combine(y, ros, top_k, wn)
        assert np.abs(out - ref).max() <= tol * max(np.abs(ref).max(), 1e-30)


@pytest.mark.gpu
def test_moe_autograd_matches_oracle_adjoints():
    from gpu_ragged_dot_amd import moe
    rng = np.random.default_rng(5)
    tokens, top_k, g, d = 50, 4, 9, 264
    ids = _random_ids(31, tokens, top_k, g, 0.1)
    _, ros, sor = moe_oracle.route(ids, g)
    h = oracle.round_to(rng.standard_normal((tokens, d)).astype(np.float32), "bfloat16")
    w = rng.random((tokens, top_k)).astype(np.float32)
    dout = oracle.round_to(rng.standard_normal((tokens, d)).astype(np.float32), "bfloat16")
    r = moe.route(torch.from_numpy(ids).cuda(), g)
    hd = util.bf16_dev(h).requires_grad_(True)
    wd = torch.from_numpy(w).cuda().requires_grad_(True)
    x = moe.dispatch(hd, r)
    out = moe.combine(x, r, wd)  # dispatch then combine: out[t] = (sum of kept weights of t) * h[t]
    out.backward(util.bf16_dev(dout))
    x_np = moe_oracle.dispatch(h, sor, top_k)
    ref_out = moe_oracle.combine(x_np, ros, top_k, w)
    assert np.abs(util.to_np(out) - ref_out).max() <= 2.0 ** -7 * np.abs(ref_out).max()
    dw_ref = moe_oracle.combine_wgrad(x_np, dout, ros, top_k)
    assert np.abs(wd.grad.cpu().numpy().reshape(tokens, top_k) - dw_ref).max() <= 1e-4 * np.abs(dw_ref).max()
    dx_ref = oracle.round_to(moe_oracle.dispatch(dout, sor, top_k, row_scale=w), "bfloat16")  # rounded once, as on the GPU
    dh_ref = moe_oracle.combine(dx_ref, ros, top_k)
    assert np.abs(util.to_np(hd.grad) - dh_ref).max() <= 2.0 ** -7 * np.abs(dh_ref).max()


@pytest.mark.gpu
def test_routed_ragged_dot_end_to_end():
    """route -> dispatch -> ragged_dot -> combine equals the dense definition sum_s w[t,s] * h[t] @ W[e(t,s)]."""
    import gpu_ragged_dot_amd as rd
    from gpu_ragged_dot_amd import moe
    rng = np.random.default_rng(9)
    tokens, top_k, g, d, n = 96, 2, 6, 128, 72
    ids = _random_ids(41, tokens, top_k, g, 0.0)
    h = oracle.round_to(rng.standard_normal((tokens, d)).astype(np.float32), "bfloat16")
    W = oracle.round_to((rng.standard_normal((g, d, n)) / d ** 0.5).astype(np.float32), "bfloat16")
    w = rng.random((tokens, top_k)).astype(np.float32)
    r = moe.route(torch.from_numpy(ids).cuda(), g)
    y = rd.ragged_dot(moe.dispatch(util.bf16_dev(h), r), util.bf16_dev(W), r.group_sizes)
    out = util.to_np(moe.combine(y, r, torch.from_numpy(w).cuda()))
    ref = np.zeros((tokens, n))
    for t in range(tokens):
        for s in range(top_k):
            ref[t] += w[t, s] * oracle.round_to((h[t].astype(np.float64) @ W[ids[t, s]].astype(np.float64)).astype(np.float32), "bfloat16")
    assert np.abs(out - ref).max() <= 1e-2 * np.abs(ref).max()
