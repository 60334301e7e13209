"""Tile-plan sweep for one problem shape on the GPU at hand - the counterpart of the reference's tuning.py, which
sweeps block_m/k/n in {32,64,128,256} with tune_jax (tuning.py:49-58).  Here the search space is the set of compiled
tile variants times the tile-walk block shape; the winners go into the planner's table.

  python -m gpu_ragged_dot_amd.tune --m 8192 --k 7168 --n 2048 --g 32 [--ops gmm,gmm_t,tgmm] [--write]
  python -m gpu_ragged_dot_amd.tune --workload mixtral_fwd_bwd --write

Group sizes for --m/--k/--n/--g follow tuning.py:41-45 (softmax of N(0,1) scaled to m, residue into the largest).
"""

from __future__ import annotations

import argparse
import json
import statistics

import numpy as np
import torch

from . import _capi, ops, planner, workloads

_HP = dict(block_m=64, block_k=64, block_n=64, interpret=False, compute_dtype=None, acc_dtype=torch.float32, chunk_m=512)


def _time_ms(fn, reps: int) -> float:
    for _ in range(2):
        fn()
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(reps):
        fn()
    stop.record()
    stop.synchronize()
    return start.elapsed_time(stop) / reps


def softmax_group_sizes(seed: int, g: int, m: int) -> np.ndarray:
    z = np.random.default_rng(seed).normal(size=g)
    e = np.exp(z - z.max())
    gs = np.round(m * e / e.sum()).astype(np.int32)
    gs[np.argmax(gs)] += m - int(gs.sum())
    return gs


def sweep(x, A, dout, gs, op: int, reps: int = 10, rounds: int = 3):
    """Median time of every (variant, walk) candidate for one product; returns a list sorted fastest first."""
    m, k = x.shape
    g = A.shape[0]
    n = A.shape[2]
    vec = k % 8 == 0 and n % 8 == 0
    # gmm: (most row tiles per band, columns per block); the product is what one XCD is dealt at a time, 32 tiles suit
    # one work-group per compute unit.  tgmm: (row tiles per band, 1 = groups visited by falling size class, -1 = as they come).
    walks = [(0, 0), (1, 32), (2, 16), (4, 8), (8, 4), (2, 4), (4, 4)] if op != _capi.OP_TGMM else [(1, -1), (2, -1), (4, -1), (8, -1), (16, -1), (4, 1), (8, 1)]
    cands = []
    for v in planner.compiled_variants():
        if bool(v.vec) != vec or v.dtype != _capi.RD_DTYPE_BF16:
            continue
        if min(m, 1 << 30) < v.tile_m // 4 and v.tile_m > 64:
            continue
        for gm, gn in walks:
            cands.append((v.name.decode(), gm, gn))
    times = {c: [] for c in cands}
    for _ in range(rounds):  # interleave the candidates: the clock under load drifts with temperature and power
        for c in cands:
            plan = _capi.Plan(planner.variant_id(c[0]), c[1], 0, c[2])
            try:
                if op == _capi.OP_GMM:
                    fn = lambda: ops._gmm_fwd(x, A, gs, **_HP, trans_rhs=False, plan=plan)
                elif op == _capi.OP_GMM_TRANS:
                    fn = lambda: ops._gmm_fwd(dout, A, gs, **_HP, trans_rhs=True, plan=plan)
                else:
                    fn = lambda: ops._tgmm_fwd(x, dout, gs, **_HP, plan=plan)
                times[c].append(_time_ms(fn, reps))
            except _capi.RaggedDotError:
                times[c].append(float("inf"))
    ranked = sorted(((statistics.median(t), c) for c, t in times.items()), key=lambda r: r[0])
    return ranked


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--workload", choices=sorted(workloads.WORKLOADS), default=None)
    ap.add_argument("--m", type=int, default=8192)  # tuning.py:31-32
    ap.add_argument("--k", type=int, default=7168)
    ap.add_argument("--n", type=int, default=2048)
    ap.add_argument("--g", type=int, default=32)
    ap.add_argument("--ops", default="gmm,gmm_t,tgmm")
    ap.add_argument("--write", action="store_true", help="merge the winners into " + planner.TUNED_PLANS_PATH)
    args = ap.parse_args()

    if args.workload:
        x, A, dout, gs = workloads.make_inputs(args.workload)
        if dout is None:
            dout = torch.randn((x.shape[0], A.shape[2]), device="cuda").to(torch.bfloat16)
    else:
        gen = torch.Generator(device="cuda").manual_seed(0)
        x = torch.randn((args.m, args.k), generator=gen, device="cuda").to(torch.bfloat16)
        A = (torch.randn((args.g, args.k, args.n), generator=gen, device="cuda") / args.k ** 0.5).to(torch.bfloat16)
        dout = torch.randn((args.m, args.n), generator=gen, device="cuda").to(torch.bfloat16)
        gs = torch.from_numpy(softmax_group_sizes(0, args.g, args.m)).cuda()
    m, k = x.shape
    g, _, n = A.shape
    flops = 2.0 * float(gs.sum().item()) * k * n
    table = {}
    for name, op, dims in (("gmm", _capi.OP_GMM, (m, k, n)), ("gmm_t", _capi.OP_GMM_TRANS, (m, n, k)),
                           ("tgmm", _capi.OP_TGMM, (m, k, n))):
        if name not in args.ops.split(","):
            continue
        ranked = sweep(x, A, dout, gs, op)
        print(f"== {name}  m={m} k={k} n={n} g={g}")
        for ms, (vname, gm, gn) in ranked[:6]:
            print(f"   {ms:8.3f} ms  {flops / ms / 1e9:8.1f} TFLOP/s   {vname} group_m={gm} group_n={gn}")
        best = ranked[0][1]
        entry = {"variant": best[0], "group_m": best[1]}
        if op != _capi.OP_TGMM or best[2]:
            entry["group_n"] = best[2]
        table[planner.plan_key(op, dims[0], dims[1], dims[2], g)] = entry
    print(json.dumps(table, indent=2))
    if args.write:
        merged = dict(planner.tuned_plans())
        merged.update(table)
        with open(planner.TUNED_PLANS_PATH, "w") as f:
            json.dump(merged, f, indent=2, sort_keys=True)
        print("written", planner.TUNED_PLANS_PATH)


if __name__ == "__main__":
    main()
