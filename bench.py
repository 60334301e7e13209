"""Throughput of the ragged_dot hot path on one MI355X.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--only] [--no-cpu-baseline]

One step = one pass of the hot path over one synthetic batch already resident in HBM: forward for the forward-only
workloads, forward + dlhs + drhs for the others.  Prints ONE JSON line.  Its top-level keys describe the headline
workload (default: the Mixtral-8x7B-shaped forward+backward).  Unless --only is given, the same line also carries
  "configs": the other measured configurations (mixtral_fwd, deepseek_fwd_bwd, decode), each with ms_per_step, value,
             roofline and cpu_baseline of its own;
  "context": what the same box does with a dense bf16 GEMM of the Mixtral forward's size (torch.matmul and this
             library's own kernels with one group, on N(0,1) data and on zeros), a sustained (>= 2 s) loop of the headline step, a bare read of the decode shape's
             bytes, the decode shape with its weights stored [g, n, k] (trans_rhs), the Mixtral-shaped products on float8
             operands, and the CPU model.
"""

import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2516.6  # dense bf16 MFMA: 256 CU x 4 SIMD x 1024 FLOP/clk x 2.4 GHz
PEAK_HBM_GBS = 8000.0
DEFAULT_WORKLOAD = "mixtral_fwd_bwd"
OTHER_CONFIGS = ("mixtral_fwd", "deepseek_fwd_bwd", "decode")
HP = dict(block_m=64, block_k=64, block_n=64, interpret=False, compute_dtype=None, chunk_m=512)


def _event_ms(fn, reps, torch):
    """Average milliseconds per call of fn() over `reps` back-to-back calls, by events on the launch stream (every
    kernel of the library is enqueued on torch's current stream, which is the one the events are recorded on)."""
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(reps):
        fn()
    stop.record()
    stop.synchronize()
    return start.elapsed_time(stop) / reps


def cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_baseline(name, seconds_hint):
    """The numpy oracle on this host's cores, on a bounded sample of the same workload: whole groups (all their rows,
    the full k and n), forward (+ backward where the workload has one), until about `seconds_hint` of work is done."""
    import numpy as np

    from gpu_ragged_dot_amd import workloads
    from oracle import ragged_dot_oracle as oracle

    w = workloads.WORKLOADS[name]
    gs = workloads.group_sizes(name)
    order = [i for i in np.argsort(-gs) if gs[i] > 0]
    rng = np.random.default_rng(0)
    done_flops, done_bytes, elapsed, used = 0.0, 0.0, 0.0, []
    for gi in order:
        rows = int(gs[gi])
        x = oracle.round_to(rng.standard_normal((rows, w.k), dtype=np.float32), "bfloat16")
        A = oracle.round_to(rng.standard_normal((1, w.k, w.n), dtype=np.float32) / np.sqrt(w.k), "bfloat16")
        one = np.array([rows], np.int32)
        t0 = time.perf_counter()
        oracle.gmm(x, A, one)
        if w.backward:
            dout = x[:, :1] * np.ones((1, w.n), np.float32)
            oracle.gmm_vjp(x, A, one, dout)
        elapsed += time.perf_counter() - t0
        done_flops += 2.0 * rows * w.k * w.n * (3 if w.backward else 1)
        done_bytes += w.k * w.n * 2
        used.append(int(gi))
        if elapsed >= seconds_hint or len(used) >= 64:
            break
    cores = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
    if name == "decode":
        value, unit = done_bytes / elapsed / 1e9, "GB/s"
    else:
        value, unit = done_flops / elapsed / 1e12, "TFLOP/s"
    return {
        "value": value,
        "unit": unit,
        "cores": cores,
        "cpu": cpu_model(),
        "kind": "port",
        "sample": f"numpy oracle (fp32 BLAS per group) on {len(used)} whole group(s) of '{name}' "
                  f"({sum(int(gs[i]) for i in used)} rows), {elapsed:.1f} s",
    }


def _plan_text(plan, planner):
    if plan.decode_nb:
        return "decode_rows" if plan.decode_nb < 0 else "decode_nb%d" % plan.decode_nb
    return "%s:%d:%d" % (planner.compiled_variants()[plan.variant].name.decode(), plan.group_m, plan.group_n)


def measure(name, steps, warmup, torch, sustained_seconds=0.0, headline=False):
    """One workload: inputs on the device, `warmup` untimed steps, then exactly `steps` timed steps between events;
    per-product launch durations and the roofline of the dominant one."""
    import gpu_ragged_dot_amd  # noqa: F401
    from gpu_ragged_dot_amd import ops, planner, workloads

    w = workloads.WORKLOADS[name]
    dev = torch.device("cuda:0")
    x, A, dout, gs = workloads.make_inputs(name, device=dev)
    hp = dict(HP, acc_dtype=torch.float32)
    if name == "decode" and not headline:  # a 35 us step: more of them (the headline keeps exactly the steps it was given)
        steps, warmup = max(steps * 10, 200), max(warmup, 20)

    # For the memory-bound decode shape the 167 MB of expert weights would otherwise sit in the 256 MB last-level
    # cache between steps: rotate over several copies so that every step streams from HBM.
    copies = [A] + ([A.clone() for _ in range(5)] if name == "decode" else [])
    state = {"i": 0}

    def fwd():
        a = copies[state["i"] % len(copies)]
        state["i"] += 1
        return ops._gmm_fwd(x, a, gs, **hp, trans_rhs=False)

    def dlhs():
        return ops._gmm_fwd(dout, A, gs, **hp, trans_rhs=True)

    def drhs():
        return ops._tgmm_fwd(x, dout, gs, **hp)

    parts = [("fwd", fwd)] + ([("dlhs", dlhs), ("drhs", drhs)] if w.backward else [])

    def step():
        for _, fn in parts:
            fn()

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    ms_per_step = _event_ms(step, steps, torch)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0

    # The decode step is one ~35 us call: also time it replayed from a HIP graph, which takes the host's launch path out
    # of the measurement.  One graph = four passes over the weight copies, 24 calls: a serving loop's graph holds a whole
    # decode step of many such calls, and the few microseconds between two replays are shared by all of them.
    graph_ms = None
    if name == "decode":
        per_graph = 4 * len(copies)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for _ in range(4):
                for a in copies:
                    ops._gmm_fwd(x, a, gs, **hp, trans_rhs=False)
        for _ in range(3):
            graph.replay()
        graph_ms = _event_ms(graph.replay, max(steps // per_graph, 4), torch) / per_graph

    # per-product launch durations, for the roofline of the dominant kernel
    if len(parts) == 1:  # the step is that one product: the timed region already is its launch duration
        per = {parts[0][0]: ms_per_step}
    else:
        per = {}
        for pname, fn in parts:
            for _ in range(2):  # the other products ran last: let this one's operands and code settle first
                fn()
            per[pname] = _event_ms(fn, max(steps, 5), torch)
    dominant = max(per, key=per.get)
    flops_step = workloads.flops(name)
    abytes = workloads.algorithmic_bytes(name)
    flops_one = flops_step / (3 if w.backward else 1)

    if name == "decode":
        metric, unit = "ragged_dot decode forward, expert weights streamed", "GB/s"
        value = abytes["weights_read"] / (ms_per_step * 1e-3) / 1e9
        roof = {"bound": "hbm", "achieved": abytes[dominant] / (per[dominant] * 1e-3) / 1e9, "peak": PEAK_HBM_GBS,
                "unit": "GB/s"}
    else:
        metric, unit = ("ragged_dot fwd+bwd" if w.backward else "ragged_dot fwd") + " throughput", "TFLOP/s"
        value = flops_step / (ms_per_step * 1e-3) / 1e12
        t_flop = flops_one / (PEAK_BF16_TFLOPS * 1e12)
        t_byte = abytes[dominant] / (PEAK_HBM_GBS * 1e9)
        if t_byte > t_flop:
            roof = {"bound": "hbm", "achieved": abytes[dominant] / (per[dominant] * 1e-3) / 1e9, "peak": PEAK_HBM_GBS,
                    "unit": "GB/s"}
        else:
            roof = {"bound": "mfma", "achieved": flops_one / (per[dominant] * 1e-3) / 1e12, "peak": PEAK_BF16_TFLOPS,
                    "unit": "TFLOP/s"}
    roof["frac"] = roof["achieved"] / roof["peak"]

    plans = {}
    for pname, op, (mm, kk, nn) in (("fwd", 0, (w.m, w.k, w.n)), ("dlhs", 1, (w.m, w.n, w.k)), ("drhs", 2, (w.m, w.k, w.n))):
        if pname in per:
            plans[pname] = _plan_text(planner.select_plan(op, mm, kk, nn, w.g), planner)

    # HBM bytes per launch of the dominant kernel, from the committed counter runs (profiles/hbm_traffic.json).  Each
    # figure there is tagged with the plan it was measured under; a figure for another plan is stale and not reported.
    roof["traffic"] = None
    try:
        with open(os.path.join(ROOT, "profiles", "hbm_traffic.json")) as f:
            entry = json.load(f).get(name, {}).get(dominant)
        if isinstance(entry, dict) and entry.get("plan") == plans.get(dominant):
            roof["traffic"] = entry.get("bytes")
    except (OSError, ValueError):
        pass
    roof["kernel"] = {"fwd": "gmm_kernel<.., trans_rhs=false>" if name != "decode" else "gmm_rows_kernel + gmm_rows_finish_kernel",
                      "dlhs": "gmm_kernel<.., trans_rhs=true>", "drhs": "tgmm_kernel"}[dominant]
    roof["launch_ms"] = per[dominant]
    roof["algorithmic_per_launch"] = abytes[dominant] if roof["bound"] == "hbm" else flops_one

    out = {
        "metric": metric,
        "value": value,
        "unit": unit,
        "ms_per_step": ms_per_step,
        "steps": steps,
        "warmup": warmup,
        "config": {"workload": name, "m": w.m, "k": w.k, "n": w.n, "g": w.g, "backward": w.backward,
                   "description": w.description, "group_sizes": "seeded, see gpu_ragged_dot_amd/workloads.py"},
        "frac_of_bf16_mfma_peak": (value / PEAK_BF16_TFLOPS) if unit == "TFLOP/s" else None,
        "frac_of_step_roofline": None,
        "per_kernel_ms": per,
        "graph_replay_ms_per_step": graph_ms,
        "tile_plans": plans,
        "wall_s_timed_region": wall,
        "roofline": roof,
    }
    if unit == "TFLOP/s":
        # time the whole step would take at max(matrix-core roof, HBM roof) of each product
        ideal = sum(max(flops_one / (PEAK_BF16_TFLOPS * 1e12), abytes[p] / (PEAK_HBM_GBS * 1e9)) for p in per)
        out["frac_of_step_roofline"] = ideal * 1e3 / ms_per_step
    if sustained_seconds > 0:
        # the same step for at least `sustained_seconds`: batches of `steps`, median and best batch
        batches, t_end = [], time.perf_counter() + sustained_seconds
        while time.perf_counter() < t_end or len(batches) < 3:
            batches.append(_event_ms(step, steps, torch))
        out["sustained"] = {"seconds": sustained_seconds, "batches": len(batches), "steps_per_batch": steps,
                            "median_ms_per_step": statistics.median(batches), "min_ms_per_step": min(batches)}
    if name == "decode":
        out["bare_stream"] = bare_stream(copies, abytes["weights_read"], torch)
        # the same experts with their weights stored [g, n, k] (trans_rhs): context, not the metric's configuration
        copies_t = [a.transpose(1, 2).contiguous() for a in copies]
        del copies[1:]

        def fwd_t():
            a = copies_t[state["i"] % len(copies_t)]
            state["i"] += 1
            return ops._gmm_fwd(x, a, gs, **hp, trans_rhs=True)

        for _ in range(max(warmup, 6)):
            fwd_t()
        ms_t = _event_ms(fwd_t, max(steps, 60), torch)
        out["trans_rhs"] = {"what": "same shape, weights stored [g, n, k] (trans_rhs=True): one launch, no workspace",
                            "us": ms_t * 1e3, "GB/s": abytes["weights_read"] / (ms_t * 1e-3) / 1e9,
                            "plan": _plan_text(planner.select_plan(1, w.m, w.k, w.n, w.g), planner)}
        del copies_t
    del x, A, dout, copies
    torch.cuda.empty_cache()
    return out


def bare_stream(copies, nbytes, torch):
    """A load-only kernel over as many bytes as the decode step streams (same rotation over weight copies), cut into
    contiguous blocks of several sizes: the floor for a transfer this small on this box."""
    from gpu_ragged_dot_amd import _capi

    out = {}
    stream = torch.cuda.current_stream().cuda_stream
    for kib in (64, 128, 256, 352):
        state = {"i": 0}

        def read():
            a = copies[state["i"] % len(copies)]
            state["i"] += 1
            _capi.check(_capi.lib.rd_probe_stream_read(stream, a.data_ptr(), nbytes, kib * 1024, None))

        for _ in range(12):
            read()
        ms = _event_ms(read, 120, torch)
        out["block_%dKiB" % kib] = {"us": ms * 1e3, "GB/s": nbytes / (ms * 1e-3) / 1e9}
    return out


def dense_gemm_context(torch):
    """hipBLASLt (torch.matmul) on dense bf16 GEMMs with the FLOPs of one Mixtral product, on N(0,1) data and on zeros:
    what the vendor library reaches on this box, and how much the data (power) matters.  Three operand layouts, those
    of the three products: forward x[m,k].W[k,n]; dlhs dout[m,n].W[k,n]^T (both operands run along the contraction
    index); drhs x[m,k]^T.dout[m,n].  Returns that and, second, this library's own kernels on the same operands."""
    from gpu_ragged_dot_amd import ops

    m, k, n = 16384, 4096, 14336
    gen = torch.Generator(device="cuda").manual_seed(7)
    out, own = {}, {}
    for label in ("normal", "zeros"):
        if label == "normal":
            a = torch.randn((m, k), generator=gen, device="cuda").to(torch.bfloat16)
            b = (torch.randn((k, n), generator=gen, device="cuda") / k ** 0.5).to(torch.bfloat16)
            d = torch.randn((m, n), generator=gen, device="cuda").to(torch.bfloat16)
        else:
            a = torch.zeros((m, k), dtype=torch.bfloat16, device="cuda")
            b = torch.zeros((k, n), dtype=torch.bfloat16, device="cuda")
            d = torch.zeros((m, n), dtype=torch.bfloat16, device="cuda")
        c = torch.empty((m, n), dtype=torch.bfloat16, device="cuda")
        ca = torch.empty((m, k), dtype=torch.bfloat16, device="cuda")
        cb = torch.empty((k, n), dtype=torch.bfloat16, device="cuda")
        layouts = (("", lambda: torch.matmul(a, b, out=c)), ("_dlhs_layout", lambda: torch.matmul(d, b.t(), out=ca)),
                   ("_drhs_layout", lambda: torch.matmul(a.t(), d, out=cb)))
        for suffix, fn in layouts:
            for _ in range(5):
                fn()
            ms = _event_ms(fn, 30, torch)
            out[label + suffix] = {"ms": ms, "TFLOP/s": 2.0 * m * k * n / (ms * 1e-3) / 1e12}
        # this library's kernels on the very same operands as ONE group of m rows (a dense GEMM through the product
        # code, default plans): the gap to the vendor kernel per layout, and zeros against N(0,1) (the power limit)
        one = torch.tensor([m], dtype=torch.int32, device="cuda")
        b3 = b.unsqueeze(0)
        hp = dict(HP, acc_dtype=torch.float32)
        own_layouts = (("", lambda: ops._gmm_fwd(a, b3, one, **hp, trans_rhs=False)),
                       ("_dlhs_layout", lambda: ops._gmm_fwd(d, b3, one, **hp, trans_rhs=True)),
                       ("_drhs_layout", lambda: ops._tgmm_fwd(a, d, one, **hp)))
        for suffix, fn in own_layouts:
            for _ in range(3):
                fn()
            ms = _event_ms(fn, 20, torch)
            own[label + suffix] = {"ms": ms, "TFLOP/s": 2.0 * m * k * n / (ms * 1e-3) / 1e12}
        del a, b, d, c, ca, cb, b3
    own["what"] = ("this library (ops._gmm_fwd / _tgmm_fwd, default plans) on the same operands as one group of 16384 "
                   "rows: forward, trans_rhs (dlhs layout), tgmm (drhs layout)")
    return {"what": "torch.matmul bf16, m16384 k4096 n14336: x.W (the Mixtral forward's FLOPs as one dense GEMM), "
                    "dout.W^T (dlhs layout), x^T.dout (drhs layout)", **out}, own


def tile_boundary_context(torch):
    """What everything between two tiles of a compute unit costs (epilogue, the next work-group's look-ups and prologue,
    the ring filling up again): the FLOPs of one dense Mixtral product as ONE group of 16384 rows on N(0,1) data, with
    the contraction lengthened and the output narrowed so that a compute unit runs 4 (14 for the forward layout), 2 (4)
    or a single 256 x 256 tile.  With one tile per compute unit there are no boundaries left: the difference to the
    first column bounds what a persistent tile-to-tile schedule could gain on this data."""
    from gpu_ragged_dot_amd import _capi, ops, planner

    m = 16384
    gen = torch.Generator(device="cuda").manual_seed(3)
    vid = planner.variant_id("w256x256x32_w2x2_s5")
    plan = _capi.Plan(vid, 4, 0, 8, -1)
    one = torch.tensor([m], dtype=torch.int32, device="cuda")
    out = {"what": "w256x256x32_w2x2_s5, one group of 16384 rows, 1.924e12 FLOP per launch, N(0,1) data, K-split off; "
                   "key = tiles per compute unit"}
    shapes = {"dlhs_layout": (True, ((14336, 4096), (28672, 2048), (57344, 1024))),
              "forward_layout": (False, ((4096, 14336), (14336, 4096), (57344, 1024)))}
    for label, (trans, kns) in shapes.items():
        res = {}
        for k, n in kns:
            x = torch.randn((m, k), generator=gen, device="cuda").to(torch.bfloat16)
            a = (torch.randn((1, n, k) if trans else (1, k, n), generator=gen, device="cuda") / k ** 0.5).to(torch.bfloat16)
            fn = lambda: ops._gmm_fwd(x, a, one, **HP, acc_dtype=torch.float32, trans_rhs=trans, plan=plan)
            for _ in range(3):
                fn()
            ms = _event_ms(fn, 10, torch)
            res[str((m // 256) * (n // 256) // 256)] = {"k": k, "n": n, "ms": ms, "TFLOP/s": 2.0 * m * k * n / (ms * 1e-3) / 1e12}
            del x, a
        out[label] = res
    return out


def schedule_context(torch):
    """The two orderings the scheduling-map kernel builds, each against the plain order on the DeepSeek-V3 workload in
    this process: gmm trans_rhs (dlhs) with the blocks of long and short groups dealt interleaved (what a call with the
    full workspace does) against the walk order (the same call through the C ABI with a workspace that holds only the
    scheduling map); tgmm (drhs) with the groups visited by falling size class (plan group_n = 1, the tuned plan) against
    the order they come in (group_n = -1)."""
    import ctypes

    from gpu_ragged_dot_amd import _capi, ops, planner, workloads

    name = "deepseek_fwd_bwd"
    x, A, dout, gs = workloads.make_inputs(name)
    w = workloads.WORKLOADS[name]
    m, k, n, g = w.m, w.k, w.n, w.g
    out = {"what": "deepseek_fwd_bwd, ms per launch"}
    # dlhs through the C ABI: y[m, k] = dout[m, n] . A[g, k, n]^T, i.e. rd_gmm(trans_rhs) with contraction n
    plan = planner.select_plan(_capi.OP_GMM_TRANS, m, n, k, g)
    y = torch.empty((m, k), dtype=torch.bfloat16, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    tile_m = [v.tile_m for v in _capi.variants() if v.id == plan.variant][0]
    units = -(-m // tile_m) + g
    map_only = -(-((g + 3 * units + 1) * 4) // 256) * 256
    full = _capi.lib.rd_gmm_workspace_bytes(m, g, ctypes.byref(plan))
    for label, nbytes in (("dlhs_blocks_interleaved", full), ("dlhs_blocks_in_walk_order", map_only)):
        ws = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
        fn = lambda: _capi.check(_capi.lib.rd_gmm(stream, dout.data_ptr(), A.data_ptr(), gs.data_ptr(), y.data_ptr(), m, n, k, g,
                                                   1, _capi.RD_DTYPE_BF16, ctypes.byref(plan), ws.data_ptr(), nbytes))
        for _ in range(3):
            fn()
        out[label] = _event_ms(fn, 20, torch)
    tuned = planner.select_plan(_capi.OP_TGMM, m, k, n, g)
    for label, gn in (("drhs_groups_by_size_class", 1), ("drhs_groups_as_they_come", -1)):
        p2 = _capi.Plan(tuned.variant, tuned.group_m, 0, gn, 0)
        fn = lambda: ops._tgmm_fwd(x, dout, gs, **HP, acc_dtype=torch.float32, plan=p2)
        for _ in range(3):
            fn()
        out[label] = _event_ms(fn, 20, torch)
    out["plans"] = {"dlhs": _plan_text(plan, planner), "drhs": _plan_text(tuned, planner)}

    # The workload taken apart: the same launches with only the groups of up to 256 rows, only the longer ones (the
    # others' sizes set to zero; the rows in use are then the first sum(group_sizes) ones - timing only), and for drhs
    # with every group empty (its 7.5 GB of stores and nothing else) beside a plain zero fill of the same tensor.
    # A launch takes about the sum of its two kinds of tiles, not their maximum.
    sizes = gs.cpu()
    short = torch.where(sizes <= 256, sizes, torch.zeros_like(sizes)).cuda()
    long_ = torch.where(sizes > 256, sizes, torch.zeros_like(sizes)).cuda()
    none = torch.zeros_like(gs)
    parts = {}
    for label, sel in (("all", gs), ("groups_up_to_256_rows", short), ("groups_over_256_rows", long_), ("no_rows", none)):
        fns = {"fwd": lambda: ops._gmm_fwd(x, A, sel, **HP, acc_dtype=torch.float32, trans_rhs=False),
               "dlhs": lambda: ops._gmm_fwd(dout, A, sel, **HP, acc_dtype=torch.float32, trans_rhs=True),
               "drhs": lambda: ops._tgmm_fwd(x, dout, sel, **HP, acc_dtype=torch.float32)}
        row = {"rows": int(sel.sum().item()), "groups": int((sel > 0).sum().item())}
        for key, fn in fns.items():
            if label == "no_rows" and key != "drhs":
                continue
            for _ in range(10):   # (the first launches after a pause run at a lower clock)
                fn()
            row[key] = _event_ms(fn, 10, torch)
        parts[label] = row
    dA = torch.empty((g, k, n), dtype=torch.bfloat16, device="cuda")
    for _ in range(3):
        dA.zero_()
    parts["zero_fill_of_the_drhs_result"] = _event_ms(lambda: dA.zero_(), 10, torch)
    out["taken_apart"] = parts
    return out


def float8_context(torch):
    """The Mixtral-shaped products with float8 e4m3fn operands (bf16 out, fp32 accumulation): forward products only - the
    library has no float8 VJP - so this is context beside the bf16 metric, not a configuration of it."""
    from gpu_ragged_dot_amd import ops, workloads

    name = "mixtral_fwd_bwd"
    x, A, dout, gs = workloads.make_inputs(name)
    w = workloads.WORKLOADS[name]
    hp = dict(block_m=64, block_k=64, block_n=64, interpret=False, compute_dtype=None, acc_dtype=torch.float32, chunk_m=512)
    x8, A8, d8 = (t.to(torch.float8_e4m3fn) for t in (x, A, dout))
    del x, A, dout
    parts = (("gmm", lambda: ops._gmm_fwd(x8, A8, gs, **hp, trans_rhs=False)),
             ("gmm_trans_rhs", lambda: ops._gmm_fwd(d8, A8, gs, **hp, trans_rhs=True)),
             ("tgmm", lambda: ops._tgmm_fwd(x8, d8, gs, **hp)))
    flops = workloads.flops(name) / 3
    out = {"what": "m16384 k4096 n14336 g8, float8 e4m3fn operands, bf16 out: x.W[g], dout.W[g]^T, x^T.dout per group"}
    for pname, fn in parts:
        for _ in range(3):
            fn()
        ms = _event_ms(fn, 20, torch)
        out[pname] = {"ms": ms, "TFLOP/s": flops / (ms * 1e-3) / 1e12, "frac_of_fp8_mfma_peak": flops / (ms * 1e-3) / 1e12 / 5033.2}
    del x8, A8, d8
    torch.cuda.empty_cache()
    return out


def bench_routing(args, torch):
    """The caller's side of the DeepSeek-V3 shaped workload: 4096 tokens x top-8 of 256 experts.  One step = route
    the (token, choice) pairs, gather the 7168-wide activations into expert order, and sum a 2048-wide product back
    per token.  HBM-bound byte work: reported as GB/s of algorithmic bytes (each tensor read or written once)."""
    from gpu_ragged_dot_amd import moe

    tokens, top_k, g, d_in, d_out = 4096, 8, 256, 7168, 2048
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    gen = torch.Generator(device=dev).manual_seed(4)
    logits = torch.randn((tokens, g), generator=gen, device=dev)
    ids = torch.topk(logits, top_k, dim=1).indices.to(torch.int32)
    wts = torch.softmax(torch.randn((tokens, top_k), generator=gen, device=dev), dim=1)
    h = torch.randn((tokens, d_in), generator=gen, device=dev).to(torch.bfloat16)
    y = torch.randn((tokens * top_k, d_out), generator=gen, device=dev).to(torch.bfloat16)
    state = {}

    def route():
        state["r"] = moe.route(ids, g)

    def dispatch():
        return moe._dispatch(h, state["r"], None)

    def combine():
        return moe._combine(y, state["r"], wts.reshape(-1))

    parts = [("route", route), ("dispatch", dispatch), ("combine", combine)]

    def step():
        for _, fn in parts:
            fn()

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    ms_per_step = _event_ms(step, args.steps, torch)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    per = {pname: _event_ms(fn, max(args.steps, 5), torch) for pname, fn in parts}
    slots = tokens * top_k
    abytes = {"route": slots * 4 * 3 + g * 4, "dispatch": (tokens + slots) * d_in * 2 + slots * 4,
              "combine": (slots + tokens) * d_out * 2 + slots * 8}
    dominant = max(per, key=per.get)
    roof = {"bound": "hbm", "achieved": abytes[dominant] / (per[dominant] * 1e-3) / 1e9, "peak": PEAK_HBM_GBS, "unit": "GB/s"}
    roof["frac"] = roof["achieved"] / roof["peak"]
    roof["traffic"] = None
    roof["kernel"] = {"route": "moe_hist/scan/rank_kernel", "dispatch": "moe_dispatch_kernel", "combine": "moe_combine_kernel"}[dominant]
    roof["launch_ms"] = per[dominant]
    out = {
        "metric": "token routing around ragged_dot (route + dispatch + combine), algorithmic bytes moved", "value": sum(abytes.values()) / (ms_per_step * 1e-3) / 1e9,
        "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "moe_routing", "tokens": tokens, "top_k": top_k, "g": g, "d_dispatch": d_in, "d_combine": d_out},
        "per_kernel_ms": per, "wall_s_timed_region": wall, "roofline": roof,
    }
    if not args.no_cpu_baseline:
        from oracle import moe_glue_oracle as mo
        ids_np, h_np, y_np, w_np = ids.cpu().numpy(), h.float().cpu().numpy(), y.float().cpu().numpy(), wts.cpu().numpy()
        t0 = time.perf_counter()
        _, ros, sor = mo.route(ids_np, g)
        mo.dispatch(h_np, sor, top_k)
        mo.combine(y_np, ros, top_k, w_np)
        dt = time.perf_counter() - t0
        out["cpu_baseline"] = {"value": sum(abytes.values()) / dt / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
                               "sample": "one whole step (numpy oracle: stable argsort, take, weighted sum)"}
    print(json.dumps(out))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default=DEFAULT_WORKLOAD)
    ap.add_argument("--only", action="store_true", help="measure the named workload only: no other configs, no context")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-seconds", type=float, default=6.0, help="CPU work per configuration for cpu_baseline")
    ap.add_argument("--sustained-seconds", type=float, default=2.0)
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain 1 GiB device copy, so a counter run has a kernel of known traffic to scale by")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.exit("bench.py measures one GPU: the ragged_dot path has no multi-GPU part; run with --gpus 1")

    import torch

    name = args.workload
    if name == "moe_routing":
        return bench_routing(args, torch)
    torch.cuda.set_device(0)
    if name == "float8_mixtral":  # the float8 entry of "context" by itself (for profiling runs)
        print(json.dumps(float8_context(torch)))
        return
    full = not args.only and name == DEFAULT_WORKLOAD and not args.copy_calibration

    if args.copy_calibration:
        src = torch.empty(1 << 30, dtype=torch.uint8, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    head = measure(name, args.steps, args.warmup, torch, sustained_seconds=args.sustained_seconds if full else 0.0, headline=True)
    out = {
        "metric": head.pop("metric"),
        "value": head.pop("value"),
        "unit": head.pop("unit"),
        "n_gpus": 1,
        "steps": head.pop("steps"),
        "warmup": head.pop("warmup"),
        "ms_per_step": head.pop("ms_per_step"),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
    }
    out.update(head)
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(name, args.cpu_seconds)
    if full:
        configs = {}
        for other in OTHER_CONFIGS:
            c = measure(other, args.steps, args.warmup, torch)
            if not args.no_cpu_baseline:
                c["cpu_baseline"] = cpu_baseline(other, args.cpu_seconds)
            configs[other] = c
        out["configs"] = configs
        vendor_dense, own_dense = dense_gemm_context(torch)
        out["context"] = {"dense_gemm": vendor_dense, "own_dense_gemm": own_dense, "sustained_headline_step": out.pop("sustained", None),
                          "decode_bare_stream": configs["decode"].pop("bare_stream", None),
                          "decode_trans_rhs": configs["decode"].pop("trans_rhs", None),
                          "tiles_per_compute_unit": tile_boundary_context(torch), "schedule_orders": schedule_context(torch),
                          "float8_mixtral_products": float8_context(torch), "cpu": cpu_model(),
                          "device": torch.cuda.get_device_name(0)}
    print(json.dumps(out))


if __name__ == "__main__":
    main()
