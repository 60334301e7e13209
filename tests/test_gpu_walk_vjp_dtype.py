"""GPU parity, second file: the tile walk as a property test, the VJP of tgmm, compute_dtype, misaligned buffers and
the K-split's workspace re-use across shapes.  Everything goes through the C ABI (ctypes) like tests/test_gpu_parity.py.
"""

import ctypes

import numpy as np
import pytest
import torch

import gpu_ragged_dot_amd as rd
from gpu_ragged_dot_amd import _capi, ops
from oracle import ragged_dot_oracle as oracle
from tests import util

pytestmark = pytest.mark.gpu

HP = dict(block_m=64, block_k=64, block_n=64, interpret=False, compute_dtype=None, acc_dtype=torch.float32, chunk_m=512)


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _bf16_variants():
    return [(v.id, v.name.decode()) for v in _capi.variants() if v.dtype == _capi.RD_DTYPE_BF16]


# ---------------------------------------------------------------------------------------------------------------------
# tile walk: any (group_m, group_n) the library accepts must visit every tile exactly once
# ---------------------------------------------------------------------------------------------------------------------

def _walk_pairs():
    rng = np.random.default_rng(12)
    pairs = [(1, 1), (1, 32), (32, 1), (1, 7), (7, 1), (4, 8), (3, 5), (127, 1), (127, 32), (2, 2048), (5, 6), (64, 64)]
    while len(pairs) < 24:
        pairs.append((int(rng.integers(1, 40)), int(rng.integers(1, 70))))
    return pairs


@pytest.mark.parametrize("vid,vname", _bf16_variants(), ids=[v[1] for v in _bf16_variants()])
def test_tile_walk_visits_every_tile_once(vid, vname):
    """A ragged shape with an empty group, a zero tail and partial last column tiles.  For every walk the output is
    NaN-poisoned first: no NaN may survive, the rows below m (guard rows) must stay untouched, the first walk must
    match the oracle and every other walk must reproduce it bit for bit (same tile arithmetic, other visiting order)."""
    m, k, n, g = 1100, 136, 520, 6
    lhs, rhs, dout, _, _ = util.make_case(21, m, k, n, g, 1.0, True, scale_rhs=True)
    gs = np.array([300, 0, 17, 450, 1, 212], np.int32)  # sum 980 < 1100: 120 tail rows
    target_m = int(gs.sum())
    x, d = util.bf16_dev(lhs), util.bf16_dev(dout)
    A, At = util.bf16_dev(rhs), util.bf16_dev(np.ascontiguousarray(np.swapaxes(rhs, 1, 2)))
    gs_d = torch.from_numpy(gs).cuda()
    y_ref = oracle.gmm(lhs, rhs, gs)
    dA_ref = oracle.tgmm(lhs, dout, gs)
    guard_rows = 64
    first = {}
    for gm, gn in _walk_pairs():
        print(f"walk {vname} group_m={gm} group_n={gn}", flush=True)
        plan = _capi.Plan(vid, gm, 0, gn, split_k=-1)
        ws = torch.empty(max(_capi.lib.rd_gmm_workspace_bytes(m, g, ctypes.byref(plan)),
                             _capi.lib.rd_tgmm_workspace_bytes(m, g, ctypes.byref(plan))), dtype=torch.uint8, device="cuda")
        for trans_rhs in (0, 1):
            buf = torch.full((m + guard_rows, n), float("nan"), dtype=torch.bfloat16, device="cuda")
            buf[m:] = 7.0
            rc = _capi.lib.rd_gmm(_stream(), x.data_ptr(), (At if trans_rhs else A).data_ptr(), gs_d.data_ptr(),
                                  buf.data_ptr(), m, k, n, g, trans_rhs, _capi.RD_DTYPE_BF16, ctypes.byref(plan),
                                  ws.data_ptr(), ws.numel())
            assert rc == 0, _capi.lib.rd_last_error()
            torch.cuda.synchronize()
            assert not torch.isnan(buf).any(), "a tile was never written"
            assert torch.all(buf[m:] == 7.0), "rows past m were touched"
            assert not torch.any(buf[target_m:m]), "tail rows must be zero"
            key = ("gmm", trans_rhs)
            if key not in first:
                first[key] = buf[:m].clone()
                util.assert_close_rows(util.to_np(buf[:m]), y_ref, target_m, util.BF16_EPS, f"y trans_rhs={trans_rhs}")
            else:
                assert torch.equal(buf[:m], first[key]), "the walk changed the result"
        out = torch.full((g, k, n), float("nan"), dtype=torch.bfloat16, device="cuda")
        rc = _capi.lib.rd_tgmm(_stream(), x.data_ptr(), d.data_ptr(), gs_d.data_ptr(), out.data_ptr(), m, k, n, g,
                               _capi.RD_DTYPE_BF16, ctypes.byref(plan), ws.data_ptr(), ws.numel())
        assert rc == 0, _capi.lib.rd_last_error()
        torch.cuda.synchronize()
        assert not torch.isnan(out).any()
        assert not torch.any(out[1]), "empty group's slice must be zero"
        if "tgmm" not in first:
            first["tgmm"] = out.clone()
            util.assert_close_groups(util.to_np(out), dA_ref, gs != 0, util.TGMM_BF16_EPS, "dA")
        else:
            assert torch.equal(out, first["tgmm"])


def test_tile_walk_rejects_what_it_cannot_serve():
    """Band heights beyond 127 row tiles or blocks beyond 4096 tiles are refused, not silently mis-walked."""
    m, k, n, g = 300, 64, 264, 3
    x = torch.zeros((m, k), dtype=torch.bfloat16, device="cuda")
    A = torch.zeros((g, k, n), dtype=torch.bfloat16, device="cuda")
    y = torch.empty((m, n), dtype=torch.bfloat16, device="cuda")
    gs = torch.tensor([100, 100, 100], dtype=torch.int32, device="cuda")
    vid = _bf16_variants()[0][0]
    for gm, gn in ((128, 1), (1000, 1), (127, 33), (64, 65), (-3, 4)):
        plan = _capi.Plan(vid, gm, 0, gn)
        ws = torch.empty(_capi.lib.rd_gmm_workspace_bytes(m, g, None), dtype=torch.uint8, device="cuda")
        rc = _capi.lib.rd_gmm(_stream(), x.data_ptr(), A.data_ptr(), gs.data_ptr(), y.data_ptr(), m, k, n, g, 0,
                              _capi.RD_DTYPE_BF16, ctypes.byref(plan), ws.data_ptr(), ws.numel())
        if gm < 0:
            assert rc == 0  # non-positive = default
        else:
            assert rc == _capi.RD_ERR_INVALID_ARGUMENT, (gm, gn, rc)
    torch.cuda.synchronize()


# ---------------------------------------------------------------------------------------------------------------------
# the VJP of tgmm (what gpu_ragged_dot.py:431-450 intends; never exercised by the reference's tests)
# ---------------------------------------------------------------------------------------------------------------------

GRID = util.reference_grid(40)


@pytest.mark.parametrize("dtype", ["bf16", "f32"])
@pytest.mark.parametrize("c", GRID[:14], ids=[util.case_id(c) for c in GRID[:14]])
def test_tgmm_vjp(c, dtype):
    """torch.autograd.grad through rd.tgmm against oracle.tgmm_vjp (pinned on the CPU by adjoint identities and central
    differences): dx_g = y_g do_g^T, dy_g = x_g do_g; rows past sum(group_sizes) get exactly zero."""
    print("tgmm vjp", dtype, c, flush=True)
    lhs, _, dout2d, gs, target_m = util.make_case(c["seed"], c["m"], c["k"], c["n"], c["g"], c["fill_in"], c["random_inputs"])
    rng = np.random.default_rng(c["seed"] + c["m"] + 3 * c["k"])
    do = rng.normal(size=(c["g"], c["k"], c["n"])).astype(np.float32)
    if dtype == "bf16":
        do = oracle.round_to(do, "bfloat16")
        dev = util.bf16_dev
        kw, eps = {}, util.BF16_EPS
    else:
        lhs = lhs + rng.normal(size=lhs.shape).astype(np.float32) * 1e-3  # not representable in bf16
        dout2d = dout2d + rng.normal(size=dout2d.shape).astype(np.float32) * 1e-3
        dev = lambda a: torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).cuda()
        kw, eps = dict(out_dtype="float32", acc=np.float64), 5e-4
    x_t, y_t = dev(lhs).requires_grad_(True), dev(dout2d).requires_grad_(True)
    out = rd.tgmm(x_t, y_t, torch.from_numpy(gs), block_m=c["block_m"], block_k=c["block_k"], block_n=c["block_n"],
                  chunk_m=c["chunk_m"])
    dx, dy = torch.autograd.grad(out, (x_t, y_t), dev(do))
    dx_ref, dy_ref, _ = oracle.tgmm_vjp(lhs, dout2d, gs, do, **kw)
    rows = np.arange(c["m"]) < target_m
    for name, got, ref in (("dx", dx, dx_ref), ("dy", dy, dy_ref)):
        got = util.to_np(got)
        assert got.shape == ref.shape
        assert float(np.max(oracle.err_fn(got, ref, mask=rows))) < eps, name
        assert float(np.max(np.abs(got - ref))) <= util.NORTH_STAR_TOL * max(float(np.max(np.abs(ref))), 1e-30), name
        assert not np.any(got[target_m:]), f"{name}: rows past sum(group_sizes) must be exactly zero"


def test_tgmm_vjp_empty_group_and_tail():
    """An empty group in the middle and unused rows at the end: the empty group's cotangent slab reaches no row."""
    m, k, n, g = 300, 72, 136, 5
    lhs, _, dout2d, _, _ = util.make_case(31, m, k, n, g, 1.0, True)
    gs = np.array([90, 0, 120, 1, 40], np.int32)  # 251 of 300 rows
    do = oracle.round_to(np.random.default_rng(31).normal(size=(g, k, n)).astype(np.float32), "bfloat16")
    x_t, y_t = util.bf16_dev(lhs).requires_grad_(True), util.bf16_dev(dout2d).requires_grad_(True)
    dx, dy = torch.autograd.grad(rd.tgmm(x_t, y_t, torch.from_numpy(gs)), (x_t, y_t), util.bf16_dev(do))
    dx_ref, dy_ref, _ = oracle.tgmm_vjp(lhs, dout2d, gs, do)
    util.assert_close_rows(util.to_np(dx), dx_ref, 251, util.BF16_EPS, "dx")
    util.assert_close_rows(util.to_np(dy), dy_ref, 251, util.BF16_EPS, "dy")
    assert not np.any(util.to_np(dx)[251:]) and not np.any(util.to_np(dy)[251:])
    do2 = do.copy()
    do2[1] = 100.0  # the empty group's cotangent must not matter
    dx2, dy2 = torch.autograd.grad(rd.tgmm(x_t, y_t, torch.from_numpy(gs)), (x_t, y_t), util.bf16_dev(do2))
    assert torch.equal(dx2, dx) and torch.equal(dy2, dy)


# ---------------------------------------------------------------------------------------------------------------------
# compute_dtype (gpu_ragged_dot.py:116-119, 145, 248, 270)
# ---------------------------------------------------------------------------------------------------------------------

def _f32_case(c):
    rng = np.random.default_rng(c["seed"] * 103 + c["m"] + c["k"] + c["n"])
    m, k, n, g = c["m"], c["k"], c["n"], c["g"]
    lhs, rhs, dout = (rng.normal(size=s).astype(np.float32) for s in ((m, k), (g, k, n), (m, n)))
    target_m = max(min(round(m * c["fill_in"]), m), 0)
    gs = oracle.generate_group_sizes(c["seed"] + 7 * g + target_m, g, target_m)
    return lhs, rhs, dout, gs, target_m


@pytest.mark.parametrize("trans_rhs", [False, True], ids=["A", "At"])
@pytest.mark.parametrize("c", GRID[:14], ids=[util.case_id(c) for c in GRID[:14]])
def test_compute_dtype_bf16_on_float32(c, trans_rhs):
    """float32 arrays with compute_dtype=bfloat16: operands rounded to bf16 (nearest even) before the dot, fp32
    accumulation, float32 out - forward and both cotangents.  The oracle does the same rounding on the host, so the
    agreement is far tighter than the bf16 eps; against the unrounded float64 product it is the bf16 eps."""
    print("compute_dtype bf16 on f32", c, "trans_rhs", trans_rhs, flush=True)
    lhs, rhs, dout, gs, target_m = _f32_case(c)
    rhs_in = np.ascontiguousarray(np.swapaxes(rhs, 1, 2)) if trans_rhs else rhs
    x_t = torch.from_numpy(lhs).cuda().requires_grad_(True)
    A_t = torch.from_numpy(rhs_in).cuda().requires_grad_(True)
    o = rd.gmm(x_t, A_t, torch.from_numpy(gs), block_m=c["block_m"], block_k=c["block_k"], block_n=c["block_n"],
               chunk_m=c["chunk_m"], trans_rhs=trans_rhs, compute_dtype=torch.bfloat16)
    assert o.dtype == torch.float32
    dlhs, drhs = torch.autograd.grad(o, (x_t, A_t), torch.from_numpy(dout).cuda())
    assert dlhs.dtype == torch.float32 and drhs.dtype == torch.float32
    r = lambda a: oracle.round_to(a, "bfloat16")
    f64 = dict(out_dtype="float32", acc=np.float64)
    o_ref = oracle.gmm(r(lhs), r(rhs_in), gs, trans_rhs=trans_rhs, **f64)
    dlhs_ref, drhs_ref, _ = oracle.gmm_vjp(r(lhs), r(rhs_in), gs, r(dout), trans_rhs=trans_rhs, **f64)
    rows = np.arange(c["m"]) < target_m
    tight = 2e-5  # fp32 accumulation of exact products against float64
    assert float(np.max(oracle.err_fn(util.to_np(o), o_ref, mask=rows))) < tight
    assert float(np.max(oracle.err_fn(util.to_np(dlhs), dlhs_ref, mask=rows))) < tight
    assert float(np.max(oracle.err_fn(util.to_np(drhs), drhs_ref, axis=(-1, -2), mask=gs != 0))) < tight
    o_full = oracle.gmm(lhs, rhs_in, gs, trans_rhs=trans_rhs, **f64)
    assert float(np.max(oracle.err_fn(util.to_np(o), o_full, mask=rows))) < util.BF16_EPS * 2
    assert not np.any(util.to_np(o)[target_m:]) and not np.any(util.to_np(dlhs)[target_m:])
    assert not np.any(util.to_np(drhs)[gs == 0])


@pytest.mark.parametrize("shape", [(1030, 264, 392, 5), (515, 99, 131, 3)], ids=lambda s: "m%d_k%d_n%d_g%d" % s)
def test_compute_dtype_every_tile_shape_and_tgmm(shape):
    """Each tile shape compiled for float32 arrays on the bf16 matrix cores, forced through the plan (the 16-byte-pitch
    one only where the shape allows it), for gmm, gmm trans_rhs and tgmm."""
    m, k, n, g = shape
    rng = np.random.default_rng(m + k)
    lhs, rhs, dout = (rng.normal(size=s).astype(np.float32) for s in ((m, k), (g, k, n), (m, n)))
    gs = oracle.generate_group_sizes(5 + m, g, m - 29)
    rows = np.arange(m) < m - 29
    r = lambda a: oracle.round_to(a, "bfloat16")
    f64 = dict(out_dtype="float32", acc=np.float64)
    o_ref = oracle.gmm(r(lhs), r(rhs), gs, **f64)
    dl_ref = oracle.gmm(r(dout), r(rhs), gs, trans_rhs=True, **f64)
    dr_ref = oracle.tgmm(r(lhs), r(dout), gs, **f64)
    x_t, A_t, d_t, gs_t = (torch.from_numpy(a).cuda() for a in (lhs, rhs, dout, gs))
    ids = [v for v in _capi.variants() if v.dtype == _capi.RD_DTYPE_F32_BF16]
    assert len(ids) >= 2
    ran = 0
    for v in ids:
        if v.vec and (k % 8 or n % 8):
            continue
        print("compute_dtype tile", v.name.decode(), shape, flush=True)
        hp = dict(HP, compute_dtype=torch.bfloat16)
        o = ops._gmm_fwd(x_t, A_t, gs_t, **hp, trans_rhs=False, plan=_capi.Plan(v.id))
        dl = ops._gmm_fwd(d_t, A_t, gs_t, **hp, trans_rhs=True, plan=_capi.Plan(v.id))
        dr = ops._tgmm_fwd(x_t, d_t, gs_t, **hp, plan=_capi.Plan(v.id))
        assert float(np.max(oracle.err_fn(util.to_np(o), o_ref, mask=rows))) < 2e-5
        assert float(np.max(oracle.err_fn(util.to_np(dl), dl_ref, mask=rows))) < 2e-5
        assert float(np.max(oracle.err_fn(util.to_np(dr), dr_ref, axis=(-1, -2), mask=gs != 0))) < 2e-5
        assert not np.any(util.to_np(o)[m - 29:]) and not np.any(util.to_np(dr)[gs == 0])
        ran += 1
    assert ran >= 1
    out = rd.tgmm(x_t, d_t, gs_t, compute_dtype=torch.bfloat16)  # default plan
    assert float(np.max(oracle.err_fn(util.to_np(out), dr_ref, axis=(-1, -2), mask=gs != 0))) < 2e-5


def test_compute_dtype_float32_on_bf16_is_the_plain_product():
    """Widening bf16 operands to float32 before the dot changes nothing (exact products, fp32 accumulation)."""
    lhs, rhs, _, gs, _ = util.make_case(3, 256, 128, 136, 4, 0.9, True, scale_rhs=True)
    x, A, gs_t = util.bf16_dev(lhs), util.bf16_dev(rhs), torch.from_numpy(gs)
    assert torch.equal(rd.gmm(x, A, gs_t, compute_dtype=torch.float32), rd.gmm(x, A, gs_t))
    with pytest.raises(NotImplementedError):
        rd.gmm(x, A, gs_t, compute_dtype=torch.float16)
    with pytest.raises(NotImplementedError):
        rd.gmm(x.float(), A.float(), gs_t, compute_dtype=torch.float16)


# ---------------------------------------------------------------------------------------------------------------------
# buffers that are contiguous but not 16-byte aligned
# ---------------------------------------------------------------------------------------------------------------------

@pytest.mark.parametrize("which", ["x", "A", "dout"])
def test_operand_view_at_an_odd_element_offset(which):
    """A contiguous view that starts 4 elements (8 bytes) into an allocation: .contiguous() is a no-op for it, the fast
    tile shapes cannot take it, and the call must fall back to the element-granular shape by itself - on a shape for
    which the tuned table / default plan would pick a 16-byte one."""
    m, k, n, g = 512, 256, 512, 4
    lhs, rhs, dout, gs, target_m = util.make_case(9, m, k, n, g, 0.9, True, scale_rhs=True)
    gs_t = torch.from_numpy(gs)

    def shifted(a):
        flat = torch.empty(a.size + 4, dtype=torch.bfloat16, device="cuda")
        view = flat[4:].view(a.shape)
        view.copy_(util.bf16_dev(a))
        assert view.is_contiguous() and view.data_ptr() % 16 == 8
        return view

    x = shifted(lhs) if which == "x" else util.bf16_dev(lhs)
    A = shifted(rhs) if which == "A" else util.bf16_dev(rhs)
    At = shifted(np.ascontiguousarray(np.swapaxes(rhs, 1, 2))) if which == "A" else util.bf16_dev(np.ascontiguousarray(np.swapaxes(rhs, 1, 2)))
    d = shifted(dout) if which == "dout" else util.bf16_dev(dout)
    y_ref = oracle.gmm(lhs, rhs, gs)
    util.assert_close_rows(util.to_np(rd.gmm(x, A, gs_t)), y_ref, target_m, util.BF16_EPS, "gmm")
    util.assert_close_rows(util.to_np(rd.gmm(x, At, gs_t, trans_rhs=True)), y_ref, target_m, util.BF16_EPS, "gmm trans_rhs")
    util.assert_close_groups(util.to_np(rd.tgmm(x, d, gs_t)), oracle.tgmm(lhs, dout, gs), gs != 0, util.TGMM_BF16_EPS, "tgmm")
    # through the bare C entry point with no plan the library picks the any-alignment shape itself
    y = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
    ws = torch.empty(_capi.lib.rd_gmm_workspace_bytes(m, g, None), dtype=torch.uint8, device="cuda")
    rc = _capi.lib.rd_gmm(_stream(), x.data_ptr(), A.data_ptr(), gs_t.cuda().data_ptr(), y.data_ptr(), m, k, n, g, 0,
                          _capi.RD_DTYPE_BF16, None, ws.data_ptr(), ws.numel())
    torch.cuda.synchronize()
    assert rc == 0, _capi.lib.rd_last_error()
    util.assert_close_rows(util.to_np(y), y_ref, target_m, util.BF16_EPS, "gmm, no plan")
    if which != "dout":
        # a forced 16-byte shape on such a buffer is refused with a status code, not a fault
        fast = [v.id for v in _capi.variants() if v.vec and v.dtype == _capi.RD_DTYPE_BF16][0]
        plan = _capi.Plan(fast)
        rc = _capi.lib.rd_gmm(_stream(), x.data_ptr(), A.data_ptr(), gs_t.cuda().data_ptr(), y.data_ptr(), m, k, n, g, 0,
                              _capi.RD_DTYPE_BF16, ctypes.byref(plan), ws.data_ptr(), ws.numel())
        assert rc == _capi.RD_ERR_UNSUPPORTED


# ---------------------------------------------------------------------------------------------------------------------
# K-split: one workspace re-used by calls of different shapes
# ---------------------------------------------------------------------------------------------------------------------

def test_k_split_workspace_reused_across_shapes():
    """The same workspace serves two problems in turn whose split tiles differ in number and in pieces per tile, so
    a slot of partial sums is re-used with another `parts`.  Each call must match its own unsplit run."""
    vid = [v.id for v in _capi.variants() if v.name.decode().startswith("q256")][0]
    shapes = [(900, 1096, 520, 5, 8), (2100, 4104, 256, 3, 3), (900, 1096, 520, 5, 2), (700, 2056, 1032, 4, 8)]
    need = max(_capi.lib.rd_gmm_workspace_bytes(s[0], s[3], ctypes.byref(_capi.Plan(vid, 2, 0, 2, split_k=8))) for s in shapes)
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    ws.fill_(0x5A)
    for m, k, n, g, parts in shapes * 2:
        print(f"k-split reuse m={m} k={k} n={n} g={g} parts<={parts}", flush=True)
        lhs, rhs, _, gs, _ = util.make_case(m + parts, m, k, n, g, 0.9, True, scale_rhs=True)
        target_m = int(gs.sum())
        x, A, gs_d = util.bf16_dev(lhs), util.bf16_dev(rhs), torch.from_numpy(gs).cuda()
        outs = []
        for plan in (_capi.Plan(vid, 2, 0, 2, split_k=parts), _capi.Plan(vid, 2, 0, 2, split_k=-1)):
            y = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
            rc = _capi.lib.rd_gmm(_stream(), x.data_ptr(), A.data_ptr(), gs_d.data_ptr(), y.data_ptr(), m, k, n, g, 0,
                                  _capi.RD_DTYPE_BF16, ctypes.byref(plan), ws.data_ptr(), ws.numel())
            assert rc == 0, _capi.lib.rd_last_error()
            torch.cuda.synchronize()
            outs.append(util.to_np(y))
        assert not np.isnan(outs[0]).any()
        util.assert_close_rows(outs[0], oracle.gmm(lhs, rhs, gs), target_m, util.BF16_EPS, "split y")
        scale = np.abs(outs[1]).max()
        assert np.abs(outs[0] - outs[1]).max() <= 2 ** -7 * scale


# ---------------------------------------------------------------------------------------------------------------------
# the streaming routines for row tiles of short groups inside the 256 x 256 four-wave kernel
# ---------------------------------------------------------------------------------------------------------------------

@pytest.mark.parametrize("trans_rhs", [False, True], ids=["A", "At"])
@pytest.mark.parametrize("k,split_k", [(72, -1), (1096, -1), (4104, 8), (2048, 3)], ids=["k72", "k1096", "k4104-split8", "k2048-split3"])
def test_short_group_row_tiles(k, split_k, trans_rhs):
    """Groups of 1..64 rows (64-row streaming routine), 65..128 rows (128-row routine), 129..256 and longer (tall
    routine, also for the short last tile of a long group) in one launch of the four-wave kernel, with contraction
    lengths that end inside a slab, and with the K-split cutting those tiles too."""
    vid = [v.id for v in _capi.variants() if v.name.decode().startswith("w256")][0]
    gs = np.array([5, 64, 65, 128, 129, 0, 33, 100, 1, 256, 300, 257, 640], np.int32)
    m, n, g = int(gs.sum()) + 40, 520, gs.size
    print(f"short tiles k={k} split_k={split_k} trans_rhs={trans_rhs}", flush=True)
    lhs, rhs, _, _, _ = util.make_case(k, m, k, n, g, 1.0, True, scale_rhs=True)
    target_m = int(gs.sum())
    x = util.bf16_dev(lhs)
    A = util.bf16_dev(np.ascontiguousarray(np.swapaxes(rhs, 1, 2)) if trans_rhs else rhs)
    gs_d = torch.from_numpy(gs).cuda()
    plan = _capi.Plan(vid, 2, 0, 4, split_k=split_k)
    ws = torch.empty(_capi.lib.rd_gmm_workspace_bytes(m, g, ctypes.byref(plan)), dtype=torch.uint8, device="cuda")
    ws.fill_(0x3C)
    y_ref = oracle.gmm(lhs, rhs, gs)
    prev = None
    for _ in range(2):
        y = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
        rc = _capi.lib.rd_gmm(_stream(), x.data_ptr(), A.data_ptr(), gs_d.data_ptr(), y.data_ptr(), m, k, n, g,
                              int(trans_rhs), _capi.RD_DTYPE_BF16, ctypes.byref(plan), ws.data_ptr(), ws.numel())
        assert rc == 0, _capi.lib.rd_last_error()
        torch.cuda.synchronize()
        assert not torch.isnan(y).any()
        util.assert_close_rows(util.to_np(y), y_ref, target_m, util.BF16_EPS, "y")
        assert not torch.any(y[target_m:])
        assert prev is None or torch.equal(prev, y)
        prev = y


@pytest.mark.parametrize("split_k", [0, -1, 2])
@pytest.mark.parametrize("n", [1728, 1792, 1800, 1864, 2048, 2584])
def test_trans_rhs_long_contraction(n, split_k):
    """gmm with trans_rhs on the four-wave variant around and above the contraction length (1792) from which its
    register-staged form takes the tall tiles: whole and partial last 64-wide slabs, row tiles with 1 .. 256 live rows,
    an empty group, a zero tail, a partial last column tile, with and without the K-split (whose pieces may fall back
    under the threshold)."""
    vid = [v.id for v in _capi.variants() if v.name.decode().startswith("w256")][0]
    gs = np.array([300, 0, 17, 260, 123, 1, 640], np.int32)
    g, k = gs.size, 520  # k: columns of the output here
    m = int(gs.sum()) + 40
    print(f"trans_rhs long contraction n={n} split_k={split_k}", flush=True)
    lhs, rhs, dout, _, _ = util.make_case(n, m, k, n, g, 1.0, True, scale_rhs=True)
    target_m = int(gs.sum())
    d = util.bf16_dev(dout)
    A = util.bf16_dev(rhs)  # [g, k, n]: with trans_rhs the contraction runs over n
    gs_d = torch.from_numpy(gs).cuda()
    plan = _capi.Plan(vid, 4, 0, 8, split_k=split_k)
    ws = torch.empty(_capi.lib.rd_gmm_workspace_bytes(m, g, ctypes.byref(plan)), dtype=torch.uint8, device="cuda")
    ws.fill_(0x5A)
    ref = oracle.gmm(dout, rhs, gs, trans_rhs=True)
    prev = None
    for _ in range(2):
        y = torch.full((m + 16, k), float("nan"), dtype=torch.bfloat16, device="cuda")
        rc = _capi.lib.rd_gmm(_stream(), d.data_ptr(), A.data_ptr(), gs_d.data_ptr(), y.data_ptr(), m, n, k, g, 1,
                              _capi.RD_DTYPE_BF16, ctypes.byref(plan), ws.data_ptr(), ws.numel())
        assert rc == 0, _capi.lib.rd_last_error()
        torch.cuda.synchronize()
        assert torch.isnan(y[m:]).all() and not torch.isnan(y[:m]).any()
        util.assert_close_rows(util.to_np(y[:m]), ref, target_m, util.BF16_EPS, "dlhs")
        assert not torch.any(y[target_m:m])
        assert prev is None or torch.equal(prev, y[:m])
        prev = y[:m]


# ---------------------------------------------------------------------------------------------------------------------
# a slice of the groups (group_offset of jax.lax.ragged_dot; an expert-parallel rank's share of the weights)
# ---------------------------------------------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", ["bf16", "f32"])
@pytest.mark.parametrize("o,gl", [(0, 9), (3, 4), (5, 4), (8, 1), (1, 1)], ids=lambda v: str(v))
def test_group_offset_forward_and_vjp(o, gl, dtype):
    """gmm / tgmm / the VJP with A holding groups [o, o + gl) of 9: against the oracle (pinned on the CPU as the product
    with the other groups' weights zero); rows of the other groups and the tail exactly zero; shards add up to the
    whole."""
    m, k, n, G = 1500, 136, 264, 9
    lhs, rhs, dout, _, _ = util.make_case(17, m, k, n, G, 1.0, True, scale_rhs=True)
    gs = np.array([300, 0, 17, 450, 1, 212, 0, 260, 90], np.int32)  # 1330 of 1500 rows
    target_m = int(gs.sum())
    if dtype == "bf16":
        dev, kw, eps = util.bf16_dev, {}, util.BF16_EPS
    else:
        rng = np.random.default_rng(3)
        lhs, rhs, dout = (a + rng.normal(size=a.shape).astype(np.float32) * 1e-3 for a in (lhs, rhs, dout))
        dev = lambda a: torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).cuda()
        kw, eps = dict(out_dtype="float32", acc=np.float64), 5e-4
    gs_t = torch.from_numpy(gs)
    off = np.concatenate([[0], np.cumsum(gs)])
    inside = np.zeros(m, bool)
    inside[off[o]:off[o + gl]] = True
    for trans_rhs in (False, True):
        print(f"group_offset o={o} gl={gl} {dtype} trans_rhs={trans_rhs}", flush=True)
        A_np = rhs[o:o + gl]
        A_in = np.ascontiguousarray(np.swapaxes(A_np, 1, 2)) if trans_rhs else A_np
        x_t, A_t = dev(lhs).requires_grad_(True), dev(A_in).requires_grad_(True)
        y = rd.gmm(x_t, A_t, gs_t, trans_rhs=trans_rhs, group_offset=o)
        dx, dA = torch.autograd.grad(y, (x_t, A_t), dev(dout))
        y_ref = oracle.gmm(lhs, A_in, gs, trans_rhs=trans_rhs, group_offset=o, **kw)
        dx_ref, dA_ref, _ = oracle.gmm_vjp(lhs, A_in, gs, dout, trans_rhs=trans_rhs, group_offset=o, **kw)
        for name, got, ref in (("y", y, y_ref), ("dx", dx, dx_ref)):
            got = util.to_np(got)
            assert float(np.max(oracle.err_fn(got, ref, mask=inside))) < eps, name
            assert not np.any(got[~inside]), f"{name}: rows of groups outside the slice (and the tail) must be zero"
        dA = util.to_np(dA)
        assert dA.shape == dA_ref.shape == A_in.shape
        assert float(np.max(oracle.err_fn(dA, dA_ref, axis=(-1, -2), mask=gs[o:o + gl] != 0))) < eps
        assert not np.any(dA[gs[o:o + gl] == 0])
    # tgmm's public keywords
    out = rd.tgmm(dev(lhs), dev(dout), gs_t, group_offset=o, num_actual_groups=gl)
    ref = oracle.tgmm(lhs, dout, gs, group_offset=o, num_actual_groups=gl, **kw)
    assert float(np.max(oracle.err_fn(util.to_np(out), ref, axis=(-1, -2), mask=gs[o:o + gl] != 0))) < eps


def test_group_offset_shards_add_up_and_bad_slices_are_refused():
    m, k, n, G = 1024, 256, 512, 8
    lhs, rhs, _, gs, target_m = util.make_case(23, m, k, n, G, 0.9, True, scale_rhs=True)
    x, A, gs_t = util.bf16_dev(lhs), util.bf16_dev(rhs), torch.from_numpy(gs)
    whole = rd.gmm(x, A, gs_t)
    parts = [rd.gmm(x, A[o:o + 2].contiguous(), gs_t, group_offset=o) for o in (0, 2, 4, 6)]
    assert torch.equal(sum(p.float() for p in parts), whole.float())  # disjoint row sets: exact
    y = torch.empty((m, n), dtype=torch.bfloat16, device="cuda")
    ws = torch.empty(_capi.lib.rd_gmm_workspace_bytes(m, G, None), dtype=torch.uint8, device="cuda")
    for o, gl in ((7, 2), (-1, 2), (0, 0), (8, 1)):
        rc = _capi.lib.rd_gmm_sharded(_stream(), x.data_ptr(), A.data_ptr(), gs_t.cuda().data_ptr(), y.data_ptr(), m, k, n,
                                      G, o, gl, 0, _capi.RD_DTYPE_BF16, None, ws.data_ptr(), ws.numel())
        assert rc == _capi.RD_ERR_INVALID_ARGUMENT, (o, gl, rc)
    plan = _capi.Plan(-1, 0, 64)  # a streaming kernel on a slice: refused
    rc = _capi.lib.rd_gmm_sharded(_stream(), x.data_ptr(), A.data_ptr(), gs_t.cuda().data_ptr(), y.data_ptr(), m, k, n, G, 2, 2,
                                  0, _capi.RD_DTYPE_BF16, ctypes.byref(plan), ws.data_ptr(), ws.numel())
    assert rc == _capi.RD_ERR_UNSUPPORTED
    torch.cuda.synchronize()
