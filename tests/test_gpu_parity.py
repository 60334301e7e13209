"""GPU parity: the HIP kernels, called through the C ABI, against the numpy oracle on the same seeded inputs.

Bars: scheduling map bit-exact; products within the reference's own per-row relative-L2 eps (tests.py:127,144,168,
183) and within max|diff| <= 1e-2 * max|ref|; tail rows and empty groups exactly zero.
"""

import ctypes

import numpy as np
import pytest
import torch

import gpu_ragged_dot_amd as rd
from gpu_ragged_dot_amd import _capi, workloads
from oracle import ragged_dot_oracle as oracle
from tests import util

pytestmark = pytest.mark.gpu


# ---------------------------------------------------------------------------------------------------------------------
# scheduling map: bit-exact
# ---------------------------------------------------------------------------------------------------------------------

def _map_cases():
    cases = []
    for name in ("tiny", "mixtral_fwd", "deepseek_fwd_bwd", "decode"):
        w = workloads.WORKLOADS[name]
        for chunk in (512, 256, 128, 64, 32, 8):
            cases.append((f"{name}-c{chunk}", workloads.group_sizes(name), w.m, chunk))
    rng = np.random.default_rng(7)
    for i in range(12):
        g = int(rng.integers(1, 40))
        m = int(rng.integers(1, 3000))
        fill = float(rng.choice([1.0, 0.7, 0.5, 0.0]))
        gs = oracle.generate_group_sizes(i, g, int(round(m * fill)))
        gs[rng.random(g) < 0.3] = 0
        cases.append((f"rand{i}", gs, m, int(rng.choice([1, 8, 64, 512]))))
    gs = rng.integers(0, 50, size=3000).astype(np.int32)  # more groups than one work-group scans at once
    cases.append(("g3000", gs, int(gs.sum()) + 17, 16))
    cases.append(("one-group", np.array([1000], np.int32), 1000, 8))
    cases.append(("all-empty", np.zeros(5, np.int32), 64, 8))
    cases.append(("m0", np.zeros(3, np.int32), 0, 8))
    return cases


@pytest.mark.parametrize("name,gs,m,chunk", _map_cases(), ids=[c[0] for c in _map_cases()])
def test_sched_map_bit_exact(name, gs, m, chunk):
    print(f"sched_map case={name} g={gs.size} m={m} chunk={chunk}", flush=True)
    offs, t2g, t2it, total = rd.make_group_metadata(torch.from_numpy(gs), m, chunk)
    ref = oracle.make_gmm_group_metadata(gs, m, chunk)
    np.testing.assert_array_equal(offs.cpu().numpy(), ref.group_offsets)
    np.testing.assert_array_equal(t2g.cpu().numpy(), ref.row_it2group)
    np.testing.assert_array_equal(t2it.cpu().numpy(), ref.row_it2it_in_group)
    assert int(total.item()) == int(ref.total_row_its)
    assert t2g.dtype == torch.int32 and t2it.dtype == torch.int32 and offs.dtype == torch.int32


# ---------------------------------------------------------------------------------------------------------------------
# the reference's test grid (tests.py:91-184), bf16
# ---------------------------------------------------------------------------------------------------------------------

GRID = util.reference_grid(40)


@pytest.mark.parametrize("c", GRID, ids=[util.case_id(c) for c in GRID])
def test_ragged_dot_grid(c):
    """tests.py:119-128 plus: the tail is exactly zero."""
    print("gmm fwd", c, flush=True)
    lhs, rhs, _, gs, target_m = util.make_case(c["seed"], c["m"], c["k"], c["n"], c["g"], c["fill_in"], c["random_inputs"])
    y = rd.gmm(util.bf16_dev(lhs), util.bf16_dev(rhs), torch.from_numpy(gs), block_m=c["block_m"], block_k=c["block_k"],
               block_n=c["block_n"], chunk_m=c["chunk_m"])
    y = util.to_np(y)
    y_ref = oracle.gmm(lhs, rhs, gs)
    util.assert_close_rows(y, y_ref, target_m, util.BF16_EPS, "y")
    assert not np.any(y[target_m:]), "rows past sum(group_sizes) must be exactly zero"
    if not c["random_inputs"]:
        assert np.all(y[:target_m] == c["k"])  # all-ones inputs: every valid output is exactly k


@pytest.mark.parametrize("trans_rhs", [False, True], ids=["A", "At"])
@pytest.mark.parametrize("c", GRID[:24], ids=[util.case_id(c) for c in GRID[:24]])
def test_ragged_dot_diff_grid(c, trans_rhs):
    """tests.py:130-171: forward and both cotangents through autograd, with A given as [g,k,n] or [g,n,k]."""
    print("gmm vjp", c, "trans_rhs", trans_rhs, flush=True)
    lhs, rhs, dout, gs, target_m = util.make_case(c["seed"], c["m"], c["k"], c["n"], c["g"], c["fill_in"], c["random_inputs"])
    rhs_in = np.ascontiguousarray(np.swapaxes(rhs, 1, 2)) if trans_rhs else rhs
    x_t = util.bf16_dev(lhs).requires_grad_(True)
    A_t = util.bf16_dev(rhs_in).requires_grad_(True)
    o = rd.gmm(x_t, A_t, torch.from_numpy(gs), block_m=c["block_m"], block_k=c["block_k"], block_n=c["block_n"],
               chunk_m=c["chunk_m"], trans_rhs=trans_rhs)
    dlhs, drhs = torch.autograd.grad(o, (x_t, A_t), util.bf16_dev(dout))
    o_ref = oracle.gmm(lhs, rhs_in, gs, trans_rhs=trans_rhs)
    dlhs_ref, drhs_ref, _ = oracle.gmm_vjp(lhs, rhs_in, gs, dout, trans_rhs=trans_rhs)
    util.assert_close_rows(util.to_np(o), o_ref, target_m, util.BF16_EPS, "o")
    util.assert_close_rows(util.to_np(dlhs), dlhs_ref, target_m, util.BF16_EPS, "dlhs")
    drhs = util.to_np(drhs)
    util.assert_close_groups(drhs, drhs_ref, gs != 0, util.BF16_EPS, "drhs")
    assert not np.any(drhs[gs == 0]), "cotangent of an empty group's weights must be exactly zero"
    assert not np.any(util.to_np(dlhs)[target_m:])


@pytest.mark.parametrize("c", GRID[:24], ids=[util.case_id(c) for c in GRID[:24]])
def test_trans_ragged_dot_grid(c):
    """tests.py:173-184."""
    print("tgmm", c, flush=True)
    lhs, _, dout, gs, _ = util.make_case(c["seed"], c["m"], c["k"], c["n"], c["g"], c["fill_in"], c["random_inputs"])
    out = rd.tgmm(util.bf16_dev(lhs), util.bf16_dev(dout), torch.from_numpy(gs), block_m=c["block_m"],
                  block_k=c["block_k"], block_n=c["block_n"], chunk_m=c["chunk_m"])
    out = util.to_np(out)
    ref = oracle.tgmm(lhs, dout, gs)
    util.assert_close_groups(out, ref, gs != 0, util.TGMM_BF16_EPS, "tgmm")
    assert not np.any(out[gs == 0])


# ---------------------------------------------------------------------------------------------------------------------
# every compiled tile shape, all three operand layouts
# ---------------------------------------------------------------------------------------------------------------------

def _variant_ids():
    return [(v.id, v.name.decode(), v.vec) for v in _capi.variants() if v.dtype == _capi.RD_DTYPE_BF16]


@pytest.mark.parametrize("vid,vname,vec", _variant_ids(), ids=[v[1] for v in _variant_ids()])
@pytest.mark.parametrize("shape", [(700, 328, 520, 5), (300, 64, 264, 3)], ids=["m700k328n520g5", "m300k64n264g3"])
def test_every_variant(vid, vname, vec, shape):
    m, k, n, g = shape
    print(f"variant {vname} shape {shape}", flush=True)
    lhs, rhs, dout, gs, target_m = util.make_case(3, m, k, n, g, 0.9, True, scale_rhs=True)
    gs[1] = 0 if g > 2 else gs[1]
    target_m = int(gs.sum())
    plan = _capi.Plan(vid, 3, 0)
    gs_t = torch.from_numpy(gs)
    hp = dict(block_m=64, block_k=64, block_n=64, interpret=False, compute_dtype=None, acc_dtype=torch.float32, chunk_m=512)
    from gpu_ragged_dot_amd import ops
    y = ops._gmm_fwd(util.bf16_dev(lhs), util.bf16_dev(rhs), gs_t, **hp, trans_rhs=False, plan=plan)
    yt = ops._gmm_fwd(util.bf16_dev(lhs), util.bf16_dev(np.ascontiguousarray(np.swapaxes(rhs, 1, 2))), gs_t, **hp,
                      trans_rhs=True, plan=plan)
    dA = ops._tgmm_fwd(util.bf16_dev(lhs), util.bf16_dev(dout), gs_t, **hp, plan=plan)
    y_ref = oracle.gmm(lhs, rhs, gs)
    util.assert_close_rows(util.to_np(y), y_ref, target_m, util.BF16_EPS, "y")
    util.assert_close_rows(util.to_np(yt), y_ref, target_m, util.BF16_EPS, "y (trans_rhs)")
    assert not np.any(util.to_np(y)[target_m:]) and not np.any(util.to_np(yt)[target_m:])
    dA_ref = oracle.tgmm(lhs, dout, gs)
    util.assert_close_groups(util.to_np(dA), dA_ref, gs != 0, util.TGMM_BF16_EPS, "dA")
    assert not np.any(util.to_np(dA)[gs == 0])


def _tall_tgmm_variants():
    return [(v.id, v.name.decode()) for v in _capi.variants()
            if v.dtype == _capi.RD_DTYPE_BF16 and v.direct_to_lds and v.tile_m == 256 and v.tile_n == 256]


@pytest.mark.parametrize("vid,vname", _tall_tgmm_variants(), ids=[v[1] for v in _tall_tgmm_variants()])
@pytest.mark.parametrize("group_m", [1, 4])
def test_tgmm_group_length_classes(vid, vname, group_m):
    """tgmm of the 256 x 256 cores on a launch with several tiles per compute unit and groups of every length class -
    empty, one slab of the K loop, two, three (the prologue's depth), more, a long one, next to each other in every
    order - with ragged edges in k and n, a zero tail, and a second call on other data."""
    from gpu_ragged_dot_amd import ops
    print(f"tgmm length classes {vname} group_m={group_m}", flush=True)
    k, n = 1288, 1544            # 6 x 7 tiles per group, the last ones partial
    lens = [0, 1, 31, 32, 33, 64, 65, 96, 97, 127, 128, 129, 160, 300, 0, 0, 7, 1100, 5, 0, 40, 200, 95, 2, 0, 64, 31, 513, 96, 33]
    rng = np.random.default_rng(11)
    gs = np.array(lens, np.int32)
    g = len(lens)
    assert g * 6 * 7 >= 4 * 256   # several tiles per compute unit
    m = int(gs.sum()) + 37
    hp = dict(block_m=64, block_k=64, block_n=64, interpret=False, compute_dtype=None, acc_dtype=torch.float32, chunk_m=512)
    plan = _capi.Plan(vid, group_m, 0)
    for scale in (1.0, -2.0):
        lhs = oracle.round_to(scale * rng.standard_normal((m, k)).astype(np.float32), "bfloat16")
        dout = oracle.round_to(rng.standard_normal((m, n)).astype(np.float32), "bfloat16")
        out = util.to_np(ops._tgmm_fwd(util.bf16_dev(lhs), util.bf16_dev(dout), torch.from_numpy(gs), **hp, plan=plan))
        ref = oracle.tgmm(lhs, dout, gs)
        util.assert_close_groups(out, ref, gs != 0, util.TGMM_BF16_EPS, f"tgmm scale={scale}")
        assert not np.any(out[gs == 0])
    # all-ones operands give every element its group's row count, exactly
    ones_x, ones_d = np.ones((m, k), np.float32), np.ones((m, n), np.float32)
    out = util.to_np(ops._tgmm_fwd(util.bf16_dev(ones_x), util.bf16_dev(ones_d), torch.from_numpy(gs), **hp, plan=plan))
    want = oracle.round_to(gs.astype(np.float32), "bfloat16")[:, None, None] * np.ones((1, k, n), np.float32)
    assert np.array_equal(out, want)


@pytest.mark.parametrize("vname", [None, "p256x256x32_w2x4_s4", "d128x128x32_w2x2_s3", "t64x64x64_w2x2"])
@pytest.mark.parametrize("g_first,g_local", [(0, 30), (7, 16)])
def test_tgmm_group_order_is_transparent(vname, g_first, g_local):
    """With plan.group_n = 1 and room for it in the workspace a tgmm launch visits the groups by falling size class.
    The same tiles are computed: the result must equal, bit for bit, that of a call whose workspace holds the row
    offsets only, and the oracle's; also for a slice of the groups (group_offset)."""
    print(f"tgmm group order {vname} groups [{g_first}, {g_first}+{g_local})", flush=True)
    k, n = 264, 520
    lens = [0, 1, 31, 32, 33, 64, 65, 96, 97, 127, 128, 129, 160, 300, 0, 0, 7, 1100, 5, 0, 40, 200, 95, 2, 0, 64, 31, 513, 96, 33]
    rng = np.random.default_rng(23)
    gs = np.array(lens, np.int32)
    g = len(lens)
    m = int(gs.sum()) + 21
    lhs = oracle.round_to(rng.standard_normal((m, k)).astype(np.float32), "bfloat16")
    dout = oracle.round_to(rng.standard_normal((m, n)).astype(np.float32), "bfloat16")
    plan = _capi.Plan(-1 if vname is None else [v.id for v in _capi.variants() if v.name.decode() == vname][0], 3, 0, 1)
    pref = ctypes.byref(plan)
    x, d, gsd = util.bf16_dev(lhs), util.bf16_dev(dout), torch.from_numpy(gs).cuda()
    full = _capi.lib.rd_tgmm_workspace_bytes(m, g, pref)
    offsets_only = -(-((g + 3 * (g + 1) + 1) * 4) // 256) * 256
    assert full >= offsets_only + 16 * g
    stream = torch.cuda.current_stream().cuda_stream
    outs = []
    for ws_bytes in (full, offsets_only):
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device="cuda")
        dA = torch.full((g_local, k, n), float("nan"), dtype=torch.bfloat16, device="cuda")
        if (g_first, g_local) == (0, g):
            rc = _capi.lib.rd_tgmm(stream, x.data_ptr(), d.data_ptr(), gsd.data_ptr(), dA.data_ptr(), m, k, n, g,
                                   _capi.RD_DTYPE_BF16, pref, ws.data_ptr(), ws_bytes)
        else:
            rc = _capi.lib.rd_tgmm_sharded(stream, x.data_ptr(), d.data_ptr(), gsd.data_ptr(), dA.data_ptr(), m, k, n, g,
                                           g_first, g_local, _capi.RD_DTYPE_BF16, pref, ws.data_ptr(), ws_bytes)
        assert rc == _capi.RD_OK, _capi.lib.rd_last_error()
        torch.cuda.synchronize()
        outs.append(dA)
    assert torch.equal(outs[0].view(torch.int16), outs[1].view(torch.int16))
    got = util.to_np(outs[0])
    sl = slice(g_first, g_first + g_local)
    util.assert_close_groups(got, oracle.tgmm(lhs, dout, gs)[sl], gs[sl] != 0, util.TGMM_BF16_EPS, "tgmm group order")
    assert not np.any(got[gs[sl] == 0])


@pytest.mark.parametrize("vname", [None, "d128x128x32_w2x2_s3", "w256x256x32_w2x2_s5"])
def test_tgmm_group_order_by_default_for_long_groups(vname):
    """plan.group_n = 0 leaves the order of the groups to the library: by size class when the groups average 512 rows
    or more, the launch has more than a round of tiles and the product is not tiny; -1 keeps the order they come in.
    Same tiles either way: equal bits, and the order records in the workspace are written only in the first case."""
    print(f"tgmm default group order {vname}", flush=True)
    k, n = 2048, 2304
    gs = np.array([900, 150, 0, 1400, 610], np.int32)
    g = len(gs)
    m = int(gs.sum()) + 12
    assert m >= 512 * g and m * k * n >= 8e9
    rng = np.random.default_rng(29)
    lhs = oracle.round_to(rng.standard_normal((m, k)).astype(np.float32), "bfloat16")
    dout = oracle.round_to(rng.standard_normal((m, n)).astype(np.float32), "bfloat16")
    vid = -1 if vname is None else [v.id for v in _capi.variants() if v.name.decode() == vname][0]
    x, d, gsd = util.bf16_dev(lhs), util.bf16_dev(dout), torch.from_numpy(gs).cuda()
    offsets_only = -(-((g + 3 * (g + 1) + 1) * 4) // 256) * 256
    stream = torch.cuda.current_stream().cuda_stream
    outs, touched = [], []
    for group_n in (0, -1, 1):
        plan = _capi.Plan(vid, 0, 0, group_n)
        ws_bytes = _capi.lib.rd_tgmm_workspace_bytes(m, g, ctypes.byref(plan))
        assert ws_bytes >= offsets_only + 16 * g
        ws = torch.full((ws_bytes,), 0xA5, dtype=torch.uint8, device="cuda")
        dA = torch.full((g, k, n), float("nan"), dtype=torch.bfloat16, device="cuda")
        rc = _capi.lib.rd_tgmm(stream, x.data_ptr(), d.data_ptr(), gsd.data_ptr(), dA.data_ptr(), m, k, n, g,
                               _capi.RD_DTYPE_BF16, ctypes.byref(plan), ws.data_ptr(), ws_bytes)
        assert rc == _capi.RD_OK, _capi.lib.rd_last_error()
        torch.cuda.synchronize()
        outs.append(dA)
        touched.append(bool((ws[offsets_only:offsets_only + 16 * g] != 0xA5).any().item()))
    assert touched == [True, False, True]
    assert torch.equal(outs[0].view(torch.int16), outs[1].view(torch.int16))
    assert torch.equal(outs[0].view(torch.int16), outs[2].view(torch.int16))
    got = util.to_np(outs[0])
    util.assert_close_groups(got, oracle.tgmm(lhs, dout, gs), gs != 0, util.TGMM_BF16_EPS, "tgmm default group order")
    assert not np.any(got[gs == 0])


@pytest.mark.parametrize("trans_rhs", [False, True], ids=["A", "At"])
@pytest.mark.parametrize("vname,walk", [("w256x256x32_w2x2_s5", (4, 8)), ("w256x256x32_w2x2_s5", (2, 4)),
                                        ("p256x256x32_w2x4_s4", (3, 5)), ("d128x128x32_w2x2_s3", (4, 8))])
def test_interleaved_block_order_is_transparent(vname, walk, trans_rhs):
    """With several rounds of tiles and room in the workspace, the blocks of the tile walk that belong to groups longer
    than the streaming routines serve are dealt interleaved with the others'.  The same tiles are computed: the result
    must equal, bit for bit, that of a call whose workspace holds the scheduling map and nothing else (blocks in walk
    order), and the oracle's within the usual bounds.  Long and short groups in every order, empty ones, a zero tail."""
    print(f"interleaved block order {vname} walk={walk} trans_rhs={trans_rhs}", flush=True)
    k, n = 72, 4096
    rng = np.random.default_rng(5)
    lens = list(rng.integers(1, 120, size=58)) + [0, 0, 0, 700, 1300, 257, 129, 128, 530]
    rng.shuffle(lens)
    gs = np.array(lens, np.int32)
    g = len(lens)
    m = int(gs.sum()) + 300
    lhs = oracle.round_to(rng.standard_normal((m, k)).astype(np.float32), "bfloat16")
    rhs = oracle.round_to((rng.standard_normal((g, k, n)) / k ** 0.5).astype(np.float32), "bfloat16")
    vid = [v.id for v in _capi.variants() if v.name.decode() == vname][0]
    bm = [v.tile_m for v in _capi.variants() if v.id == vid][0]
    plan = _capi.Plan(vid, walk[0], 0, walk[1], split_k=-1)
    x, A, gsd = util.bf16_dev(lhs), util.bf16_dev(rhs), torch.from_numpy(gs).cuda()
    Ad = A.mT.contiguous() if trans_rhs else A
    U = -(-m // bm) + g
    assert U * (n // 256) >= 1024 and (-(-gs // bm)).sum() * (n // 256) >= 1024   # several rounds of live tiles
    map_only = -(-((g + 3 * U + 1) * 4) // 256) * 256
    outs = []
    for ws_bytes in (_capi.lib.rd_gmm_workspace_bytes(m, g, ctypes.byref(plan)), map_only):
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device="cuda")
        y = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
        rc = _capi.lib.rd_gmm(torch.cuda.current_stream().cuda_stream, x.data_ptr(), Ad.data_ptr(), gsd.data_ptr(),
                              y.data_ptr(), m, k, n, g, int(trans_rhs), _capi.RD_DTYPE_BF16, ctypes.byref(plan),
                              ws.data_ptr(), ws_bytes)
        assert rc == _capi.RD_OK, _capi.lib.rd_last_error()
        torch.cuda.synchronize()
        outs.append(y)
    assert torch.equal(outs[0].view(torch.int16), outs[1].view(torch.int16))
    got = util.to_np(outs[0])
    util.assert_close_rows(got, oracle.gmm(lhs, rhs, gs), int(gs.sum()), util.BF16_EPS, "interleaved")
    assert not np.any(got[int(gs.sum()):])


def _split_variants():
    return [(v.id, v.name.decode()) for v in _capi.variants() if v.dtype == _capi.RD_DTYPE_BF16 and v.direct_to_lds]


@pytest.mark.parametrize("trans_rhs", [False, True], ids=["A", "At"])
@pytest.mark.parametrize("vid,vname", _split_variants(), ids=[v[1] for v in _split_variants()])
@pytest.mark.parametrize("shape", [(900, 1096, 520, 5), (2100, 4104, 256, 3)], ids=["m900k1096n520g5", "m2100k4104n256g3"])
def test_k_split_of_last_round(vid, vname, shape, trans_rhs):
    """Few tiles and a long contraction: the tiles are cut along K over several work-groups.  The result must match
    the oracle, agree with the unsplit run to fp32 summation order, overwrite every output element, and be the same on
    a second call that reuses the workspace (the arrival counters are cleared by every call)."""
    m, k, n, g = shape
    print(f"k-split variant {vname} shape {shape} trans_rhs {trans_rhs}", flush=True)
    lhs, rhs, _, gs, target_m = util.make_case(5, m, k, n, g, 0.9, True, scale_rhs=True)
    gs[1] = 0
    target_m = int(gs.sum())
    x = util.bf16_dev(lhs)
    A = util.bf16_dev(np.ascontiguousarray(np.swapaxes(rhs, 1, 2)) if trans_rhs else rhs)
    gs_d = torch.from_numpy(gs).cuda()
    split, whole = _capi.Plan(vid, 2, 0, 2, split_k=8), _capi.Plan(vid, 2, 0, 2, split_k=-1)  # 8: cut whatever k is
    need = _capi.lib.rd_gmm_workspace_bytes(m, g, ctypes.byref(split))
    assert need > _capi.lib.rd_gmm_workspace_bytes(m, g, ctypes.byref(whole))
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    ws.fill_(0xA5)  # stale counters and partial sums
    outs = []
    for plan in (split, split, whole):
        y = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
        rc = _capi.lib.rd_gmm(torch.cuda.current_stream().cuda_stream, x.data_ptr(), A.data_ptr(), gs_d.data_ptr(),
                              y.data_ptr(), m, k, n, g, int(trans_rhs), _capi.RD_DTYPE_BF16, ctypes.byref(plan),
                              ws.data_ptr(), ws.numel())
        torch.cuda.synchronize()
        assert rc == 0, _capi.lib.rd_last_error()
        outs.append(util.to_np(y))
    y_ref = oracle.gmm(lhs, rhs, gs)
    for y in outs:
        assert not np.isnan(y).any()
        util.assert_close_rows(y, y_ref, target_m, util.BF16_EPS, "y")
        assert not np.any(y[target_m:])
    assert np.array_equal(outs[0], outs[1])
    scale = np.abs(y_ref).max()
    assert np.abs(outs[0].astype(np.float32) - outs[2].astype(np.float32)).max() <= 2 ** -7 * scale
    # Same workspace, other data: no piece may see a partial sum of the call before (the pieces of a tile run on
    # different XCDs, whose L2 caches hold what the previous call read).  Scaling by -2 is exact in bf16 and fp32.
    x2 = (x.float() * -2.0).to(torch.bfloat16)
    y = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
    rc = _capi.lib.rd_gmm(torch.cuda.current_stream().cuda_stream, x2.data_ptr(), A.data_ptr(), gs_d.data_ptr(),
                          y.data_ptr(), m, k, n, g, int(trans_rhs), _capi.RD_DTYPE_BF16, ctypes.byref(split),
                          ws.data_ptr(), ws.numel())
    torch.cuda.synchronize()
    assert rc == 0, _capi.lib.rd_last_error()
    assert np.array_equal(util.to_np(y).astype(np.float32), -2.0 * outs[0].astype(np.float32))


@pytest.mark.parametrize("trans_rhs", [False, True], ids=["A", "At"])
@pytest.mark.parametrize("case", ["plan_cut", "long_k", "too_many", "many_groups"])
def test_short_last_tiles_move_into_the_k_split_round(case, trans_rhs):
    """Four-wave 256 x 256 core with the last round of tiles cut along K: the last row tile of a group of several row
    tiles, when it holds at most 128 rows, is listed behind all other tiles (marked in the band array of the internal
    map) and runs through the streaming routines - if all such tiles then lie in that last round.  Same bounds against
    the oracle, every element written, the same bits on a second call; without the K-split nothing moves."""
    print(f"short last tiles {case} trans_rhs {trans_rhs}", flush=True)
    if case == "plan_cut":  # cut by the plan (k itself would not ask for it)
        k, n, lens, split_k = 1096, 520, [300, 0, 520, 356, 700, 90], 8
        moved = [(0, 1), (2, 2), (3, 1)]
    elif case == "long_k":  # cut because k is long
        k, n, lens, split_k = 6664, 256, [600, 290, 0, 128], 0
        moved = [(0, 2), (1, 1)]
    elif case == "many_groups":  # more groups than the map kernel scans at a time, moved tiles in its second pass
        k, n, split_k = 1032, 128, 8
        lens = [0] * 1100
        for gi, rows in ((5, 300), (17, 64), (600, 256), (1030, 520), (1031, 128), (1090, 290), (1099, 1)):
            lens[gi] = rows
        moved = [(5, 1), (1030, 2), (1090, 1)]
    else:  # 280 tiles, a round of 256 and a last one of 24: the 140 short last tiles would not all lie in the last one
        k, n, lens, split_k = 1032, 512, [260 + i for i in range(70)], 8
        moved = []
    rng = np.random.default_rng(31)
    gs = np.array(lens, np.int32)
    g = len(lens)
    rows = int(gs.sum())
    m = rows + 13
    lhs = oracle.round_to(rng.standard_normal((m, k)).astype(np.float32), "bfloat16")
    rhs = oracle.round_to((rng.standard_normal((g, k, n)) / k ** 0.5).astype(np.float32), "bfloat16")
    x = util.bf16_dev(lhs)
    A = util.bf16_dev(np.ascontiguousarray(np.swapaxes(rhs, 1, 2)) if trans_rhs else rhs)
    gs_d = torch.from_numpy(gs).cuda()
    vid = [v.id for v in _capi.variants() if v.name.decode() == "w256x256x32_w2x2_s5"][0]
    split, whole = _capi.Plan(vid, 2, 0, 4, split_k=split_k), _capi.Plan(vid, 2, 0, 4, split_k=-1)
    need = _capi.lib.rd_gmm_workspace_bytes(m, g, ctypes.byref(split))
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    U = -(-m // 256) + g
    n_all = int(np.sum(-(-gs // 256)))
    outs, maps = [], []
    for plan in (split, split, whole):
        ws.fill_(0xA5)
        y = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
        rc = _capi.lib.rd_gmm(torch.cuda.current_stream().cuda_stream, x.data_ptr(), A.data_ptr(), gs_d.data_ptr(),
                              y.data_ptr(), m, k, n, g, int(trans_rhs), _capi.RD_DTYPE_BF16, ctypes.byref(plan),
                              ws.data_ptr(), ws.numel())
        torch.cuda.synchronize()
        assert rc == 0, _capi.lib.rd_last_error()
        outs.append(util.to_np(y))
        w = ws.view(torch.int32).cpu().numpy()
        maps.append((w[g:g + U].copy(), w[g + U:g + 2 * U].copy(), w[g + 2 * U + 1:g + 3 * U + 1].copy()))
    y_ref = oracle.gmm(lhs, rhs, gs)
    for y in outs:
        assert not np.isnan(y).any()
        util.assert_close_rows(y, y_ref, rows, util.BF16_EPS, "y")
        assert not np.any(y[rows:])
    assert np.array_equal(outs[0], outs[1])
    mark = 1 << 30
    group_of, tile_of, band = maps[0]
    assert int(np.count_nonzero(band[:n_all] & mark)) == len(moved)
    if moved:
        assert [(int(a), int(b)) for a, b in zip(group_of[n_all - len(moved):n_all], tile_of[n_all - len(moved):n_all])] == moved
        assert not np.any(band[:n_all - len(moved)] & mark)
    # every (group, row tile) pair is listed once, moved or not
    want = sorted((gi, it) for gi in range(g) for it in range(-(-int(gs[gi]) // 256)))
    assert sorted(zip(group_of[:n_all].tolist(), tile_of[:n_all].tolist())) == want
    assert not np.any(maps[2][2][:n_all] & mark)
    assert list(zip(maps[2][0][:n_all].tolist(), maps[2][1][:n_all].tolist())) == want


# ---------------------------------------------------------------------------------------------------------------------
# configuration C1 (tiny) with its exact recipe, and the other configurations' shapes
# ---------------------------------------------------------------------------------------------------------------------

def test_tiny_config_fwd_vjp():
    print("tiny config", flush=True)
    x, A, dout, gs = workloads.make_inputs("tiny")
    assert gs.cpu().tolist() == [116, 133, 132, 131]
    y, dx, dA = rd.ragged_dot_vjp(x, A, gs, dout)
    xn, An, dn, gsn = util.to_np(x), util.to_np(A), util.to_np(dout), gs.cpu().numpy()
    dx_ref, dA_ref, _ = oracle.gmm_vjp(xn, An, gsn, dn)
    util.assert_close_rows(util.to_np(y), oracle.gmm(xn, An, gsn), 512, util.BF16_EPS, "y")
    util.assert_close_rows(util.to_np(dx), dx_ref, 512, util.BF16_EPS, "dlhs")
    util.assert_close_groups(util.to_np(dA), dA_ref, gsn != 0, util.TGMM_BF16_EPS, "drhs")


def test_decode_config():
    print("decode config", flush=True)
    x, A, _, gs = workloads.make_inputs("decode")
    gsn = gs.cpu().numpy()
    assert int(gsn.sum()) == 64 and int((gsn > 0).sum()) == 53
    y_ref = oracle.gmm(util.to_np(x), util.to_np(A), gsn)
    for nb in (32, 64, 128, _capi.RD_DECODE_ROWS):   # column strips of nb, or whole-row slices
        from gpu_ragged_dot_amd import ops
        y = ops._gmm_fwd(x, A, gs, 64, 64, 64, False, False, None, torch.float32, 512, plan=_capi.Plan(-1, 0, nb))
        util.assert_close_rows(util.to_np(y), y_ref, 64, util.BF16_EPS, f"decode nb={nb}")
    y = rd.ragged_dot(x, A, gs)  # default plan for this shape is the streaming kernel
    util.assert_close_rows(util.to_np(y), y_ref, 64, util.BF16_EPS, "decode default")


def test_decode_kernel_long_groups_and_tail():
    """More rows per group than the streaming kernel holds at once, a zero tail, and a ragged last column block."""
    print("decode long groups", flush=True)
    m, k, n, g = 40, 520, 200, 6
    lhs, rhs, _, _, _ = util.make_case(5, m, k, n, g, 1.0, True, scale_rhs=True)
    gs = np.array([0, 11, 1, 0, 9, 5], np.int32)  # sum 26 < 40
    from gpu_ragged_dot_amd import ops
    for nb in (32, 64, 128, _capi.RD_DECODE_ROWS):
        y = ops._gmm_fwd(util.bf16_dev(lhs), util.bf16_dev(rhs), torch.from_numpy(gs), 64, 64, 64, False, False, None,
                         torch.float32, 512, plan=_capi.Plan(-1, 0, nb))
        y = util.to_np(y)
        util.assert_close_rows(y, oracle.gmm(lhs, rhs, gs), 26, util.BF16_EPS, f"nb={nb}")
        assert not np.any(y[26:])


@pytest.mark.parametrize("g,active,rows_each", [(600, 40, 1), (1500, 1500, 1), (300, 299, 2), (257, 3, 7)],
                         ids=["g600-sparse", "g1500-all-active", "g300-two-rows", "g257-few-long"])
def test_decode_rows_kernel_many_groups(g, active, rows_each):
    """The whole-row streaming kernel with more groups than one scan slab holds (256), and with more non-empty groups
    than it launches work-groups (each work-group then serves several experts in turn)."""
    from gpu_ragged_dot_amd import ops
    print(f"decode rows kernel g={g} active={active} rows_each={rows_each}", flush=True)
    rng = np.random.default_rng(g)
    k, n = 136, 72
    gs = np.zeros(g, np.int32)
    gs[rng.choice(g, active, replace=False)] = rows_each
    m = int(gs.sum()) + 5
    lhs = oracle.round_to(rng.standard_normal((m, k)).astype(np.float32), "bfloat16")
    rhs = oracle.round_to((rng.standard_normal((g, k, n)) / k ** 0.5).astype(np.float32), "bfloat16")
    y = ops._gmm_fwd(util.bf16_dev(lhs), util.bf16_dev(rhs), torch.from_numpy(gs), 64, 64, 64, False, False, None,
                     torch.float32, 512, plan=_capi.Plan(-1, 0, _capi.RD_DECODE_ROWS))
    y = util.to_np(y)
    util.assert_close_rows(y, oracle.gmm(lhs, rhs, gs), int(gs.sum()), util.BF16_EPS, "rows kernel")
    assert not np.any(y[int(gs.sum()):])


@pytest.mark.parametrize("k,n", [(520, 776), (2304, 200), (136, 2048)], ids=["k520-n776", "k2304-n200", "k136-n2048"])
def test_decode_rows_kernel_wide_passes(k, n):
    """More rows than groups: the whole-row streaming kernel takes up to 8 rows per pass (pairs of weight rows through
    v_dot2_f32_bf16).  Every pass height 1 .. 8, groups that need two and three passes, empty groups, a zero tail, a
    contraction longer than one staged segment, and one that is not a whole number of steps."""
    from gpu_ragged_dot_amd import ops
    print(f"decode rows kernel, wide passes k={k} n={n}", flush=True)
    gs = np.array([0, 1, 2, 3, 4, 5, 6, 7, 8, 0, 9, 12, 16, 17, 0, 3], np.int32)
    g, m = len(gs), int(gs.sum()) + 6
    rng = np.random.default_rng(k + n)
    lhs = oracle.round_to(rng.standard_normal((m, k)).astype(np.float32), "bfloat16")
    rhs = oracle.round_to((rng.standard_normal((g, k, n)) / k ** 0.5).astype(np.float32), "bfloat16")
    y = ops._gmm_fwd(util.bf16_dev(lhs), util.bf16_dev(rhs), torch.from_numpy(gs), 64, 64, 64, False, False, None,
                     torch.float32, 512, plan=_capi.Plan(-1, 0, _capi.RD_DECODE_ROWS))
    y = util.to_np(y)
    util.assert_close_rows(y, oracle.gmm(lhs, rhs, gs), int(gs.sum()), util.BF16_EPS, "rows kernel, wide passes")
    assert not np.any(y[int(gs.sum()):])


@pytest.mark.parametrize("case", ["decode-config", "long-groups-tail", "g600-sparse", "g300-two-rows", "wide-passes", "k8192", "n24"])
def test_decode_rows_kernel_trans_rhs(case):
    """Weights stored [g, n, k]: the streaming kernel that cuts every expert's weight rows into contiguous blocks along n
    and writes y in one launch.  Default plan and explicit plan, 4 and 8 rows per pass, groups that need several passes,
    empty groups, a zero tail, contraction lengths that are not a whole number of 512-element positions, more non-empty
    groups than work-groups, fewer output columns than pieces."""
    from gpu_ragged_dot_amd import ops
    print(f"decode rows kernel, trans_rhs, {case}", flush=True)
    rng = np.random.default_rng(len(case))
    if case == "decode-config":
        x, A, _, gs_t = workloads.make_inputs("decode")
        lhs, rhs, gs = util.to_np(x), util.to_np(A), gs_t.cpu().numpy()
    else:
        k, n, gs = {
            "long-groups-tail": (520, 200, np.array([0, 11, 1, 0, 9, 5], np.int32)),
            "g600-sparse": (136, 72, None),
            "g300-two-rows": (264, 40, None),
            "wide-passes": (1032, 776, np.array([0, 1, 2, 3, 4, 5, 6, 7, 8, 0, 9, 12, 16, 17, 0, 3], np.int32)),
            "k8192": (8192, 64, np.array([2, 0, 1, 3], np.int32)),
            "n24": (2048, 24, np.array([1, 0, 4, 2, 0, 0, 1, 1], np.int32)),
        }[case]
        if gs is None:
            g, active, rows_each = (600, 40, 1) if case == "g600-sparse" else (300, 299, 2)
            gs = np.zeros(g, np.int32)
            gs[rng.choice(g, active, replace=False)] = rows_each
        g, m = len(gs), int(gs.sum()) + 5
        lhs = oracle.round_to(rng.standard_normal((m, k)).astype(np.float32), "bfloat16")
        rhs = oracle.round_to((rng.standard_normal((g, k, n)) / k ** 0.5).astype(np.float32), "bfloat16")
    y_ref = oracle.gmm(lhs, rhs, gs)
    rhs_t = np.ascontiguousarray(np.swapaxes(rhs, 1, 2))  # [g, n, k]
    m = lhs.shape[0]
    live = int(min(gs.sum(), m))
    for plan in (_capi.Plan(-1, 0, _capi.RD_DECODE_ROWS), None):
        y = ops._gmm_fwd(util.bf16_dev(lhs), util.bf16_dev(rhs_t), torch.from_numpy(gs), 64, 64, 64, True, False, None,
                         torch.float32, 512, plan=plan)
        y = util.to_np(y)
        util.assert_close_rows(y, y_ref, live, util.BF16_EPS, f"trans_rhs rows kernel plan={plan}")
        assert not np.any(y[live:])


def test_decode_rows_kernel_trans_rhs_long_contraction_falls_back():
    """A contraction too long for the streaming kernel's staged activations: refused when asked for by name, and the
    default plan takes a tile kernel."""
    from gpu_ragged_dot_amd import ops
    k, n, gs = 8200, 16, np.array([1, 2], np.int32)
    rng = np.random.default_rng(1)
    lhs = oracle.round_to(rng.standard_normal((3, k)).astype(np.float32), "bfloat16")
    rhs = oracle.round_to((rng.standard_normal((2, k, n)) / k ** 0.5).astype(np.float32), "bfloat16")
    rhs_t = np.ascontiguousarray(np.swapaxes(rhs, 1, 2))
    args = (util.bf16_dev(lhs), util.bf16_dev(rhs_t), torch.from_numpy(gs), 64, 64, 64, True, False, None, torch.float32, 512)
    with pytest.raises(_capi.RaggedDotError):
        ops._gmm_fwd(*args, plan=_capi.Plan(-1, 0, _capi.RD_DECODE_ROWS))
    util.assert_close_rows(util.to_np(ops._gmm_fwd(*args)), oracle.gmm(lhs, rhs, gs), 3, util.BF16_EPS, "fallback")


# ---------------------------------------------------------------------------------------------------------------------
# what the reference leaves undefined or never checks
# ---------------------------------------------------------------------------------------------------------------------

def _raw_gmm(x, A, gs, y, trans_rhs=False, plan=None):
    m, k = x.shape
    g = A.shape[0]
    n = A.shape[1] if trans_rhs else A.shape[2]
    ws = torch.empty(_capi.lib.rd_gmm_workspace_bytes(m, g, None), dtype=torch.uint8, device="cuda")
    rc = _capi.lib.rd_gmm(torch.cuda.current_stream().cuda_stream, x.data_ptr(), A.data_ptr(), gs.data_ptr(),
                          y.data_ptr(), m, k, n, g, int(trans_rhs), _capi.RD_DTYPE_BF16,
                          ctypes.byref(plan) if plan is not None else None, ws.data_ptr(), ws.numel())
    torch.cuda.synchronize()
    return rc


@pytest.mark.parametrize("fill_in", [1.0, 0.5, 0.0])
def test_every_output_element_is_written(fill_in):
    """The output buffer arrives uninitialised (gpu_ragged_dot.py:210): poison it and require every element to be
    overwritten - including when every group is empty, which the reference leaves undefined (:157)."""
    print("poison fill_in", fill_in, flush=True)
    m, k, n, g = 300, 128, 136, 7
    lhs, rhs, _, gs, target_m = util.make_case(11, m, k, n, g, fill_in, True)
    for plan in (None, _capi.Plan(-1, 0, 64)):
        y = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
        assert _raw_gmm(util.bf16_dev(lhs), util.bf16_dev(rhs), torch.from_numpy(gs).cuda(), y, plan=plan) == 0
        y = util.to_np(y)
        assert not np.isnan(y).any()
        util.assert_close_rows(y, oracle.gmm(lhs, rhs, gs), target_m, util.BF16_EPS, "y")
        assert not np.any(y[target_m:])


def test_degenerate_shapes():
    """Empty contraction, no rows, a single narrow column block, more groups than the map kernel has threads, one
    group, every group empty: the op is defined for all of them (zeros where nothing contributes)."""
    rng = np.random.default_rng(0)
    cases = [(64, 0, 64, 4, np.array([10, 20, 4, 30], np.int32)),
             (0, 64, 64, 4, np.zeros(4, np.int32)),
             (300, 64, 8, 3, np.array([100, 50, 150], np.int32)),
             (5000, 128, 256, 3000, np.random.default_rng(1).multinomial(5000, [1 / 3000] * 3000).astype(np.int32)),
             (2048, 256, 256, 1, np.array([2048], np.int32)),
             (1024, 64, 128, 8, np.zeros(8, np.int32))]
    for m, k, n, g, gs in cases:
        print(f"degenerate m={m} k={k} n={n} g={g}", flush=True)
        x = oracle.round_to(rng.standard_normal((m, k)).astype(np.float32), "bfloat16")
        A = oracle.round_to((rng.standard_normal((g, k, n)) / max(k, 1) ** 0.5).astype(np.float32), "bfloat16")
        dout = oracle.round_to(rng.standard_normal((m, n)).astype(np.float32), "bfloat16")
        gs_t = torch.from_numpy(gs)
        y = util.to_np(rd.ragged_dot(util.bf16_dev(x), util.bf16_dev(A), gs_t))
        total = min(int(gs.sum()), m)
        assert y.shape == (m, n) and not np.any(y[total:])
        if y.size:
            ref = oracle.gmm(x, A, gs)
            assert np.abs(y - ref).max() <= 1e-2 * max(np.abs(ref).max(), 1e-30) + 0.0
        dA = util.to_np(rd.trans_ragged_dot(util.bf16_dev(x), util.bf16_dev(dout), gs_t))
        assert dA.shape == (g, k, n)
        if dA.size:
            ref = oracle.tgmm(x, dout, gs)
            assert np.abs(dA - ref).max() <= 1e-2 * max(np.abs(ref).max(), 1e-30)
            assert not np.any(dA[gs == 0])


def test_group_sizes_past_m_are_clipped():
    """sum(group_sizes) > m is out-of-bounds in the reference; here rows >= m are never touched."""
    print("clip", flush=True)
    m, k, n, g = 100, 64, 72, 4
    lhs, rhs, _, _, _ = util.make_case(2, m, k, n, g, 1.0, True)
    gs = np.array([40, 40, 40, 40], np.int32)
    guard = torch.full((m + 64, n), 7.0, dtype=torch.bfloat16, device="cuda")
    y = guard[:m]
    assert _raw_gmm(util.bf16_dev(lhs), util.bf16_dev(rhs), torch.from_numpy(gs).cuda(), y) == 0
    assert torch.all(guard[m:] == 7.0)
    clipped = np.array([40, 40, 20, 0], np.int32)
    util.assert_close_rows(util.to_np(y), oracle.gmm(lhs, rhs, clipped), m, util.BF16_EPS, "clipped y")


def test_linearity_and_group_locality():
    """Size-independent properties: scaling x by 2 scales y by exactly 2 (power of two in bf16); changing one
    group's weights changes only that group's rows."""
    print("linearity", flush=True)
    m, k, n, g = 1024, 512, 768, 8
    lhs, rhs, _, gs, _ = util.make_case(4, m, k, n, g, 1.0, True, scale_rhs=True)
    x, A, gs_t = util.bf16_dev(lhs), util.bf16_dev(rhs), torch.from_numpy(gs)
    y1 = rd.gmm(x, A, gs_t)
    y2 = rd.gmm(x * 2, A, gs_t)
    assert torch.equal(y2.float(), y1.float() * 2)
    A2 = A.clone()
    A2[3] = -A2[3]
    y3 = rd.gmm(x, A2, gs_t)
    off = np.concatenate([[0], np.cumsum(gs)])
    same = torch.ones(m, dtype=torch.bool)
    same[off[3]:off[4]] = False
    assert torch.equal(y3[same.cuda()], y1[same.cuda()])
    assert torch.equal(y3[off[3]:off[4]].float(), -y1[off[3]:off[4]].float())


# ---------------------------------------------------------------------------------------------------------------------
# float32 operands (tests.py:93 runs every test for bfloat16 and float32; eps 5e-4, tgmm 1e-4)
# ---------------------------------------------------------------------------------------------------------------------

F32_EPS, F32_TGMM_EPS = 5e-4, 1e-4


def _f32_case(c):
    rng = np.random.default_rng(c["seed"] * 101 + c["m"] + c["k"] + c["n"])
    m, k, n, g = c["m"], c["k"], c["n"], c["g"]
    if c["random_inputs"]:
        lhs, rhs, dout = (rng.normal(size=s).astype(np.float32) for s in ((m, k), (g, k, n), (m, n)))
    else:
        lhs, rhs, dout = (np.ones(s, np.float32) for s in ((m, k), (g, k, n), (m, n)))
    target_m = max(min(round(m * c["fill_in"]), m), 0)
    gs = oracle.generate_group_sizes(c["seed"] + 7 * g + target_m, g, target_m)
    return lhs, rhs, dout, gs, target_m


@pytest.mark.parametrize("trans_rhs", [False, True], ids=["A", "At"])
@pytest.mark.parametrize("c", GRID[:16], ids=[util.case_id(c) for c in GRID[:16]])
def test_float32_forward_and_vjp(c, trans_rhs):
    print("f32", c, "trans_rhs", trans_rhs, flush=True)
    lhs, rhs, dout, gs, target_m = _f32_case(c)
    rhs_in = np.ascontiguousarray(np.swapaxes(rhs, 1, 2)) if trans_rhs else rhs
    x_t = torch.from_numpy(lhs).cuda().requires_grad_(True)
    A_t = torch.from_numpy(rhs_in).cuda().requires_grad_(True)
    o = rd.gmm(x_t, A_t, torch.from_numpy(gs), block_m=c["block_m"], block_k=c["block_k"], block_n=c["block_n"],
               chunk_m=c["chunk_m"], trans_rhs=trans_rhs)
    assert o.dtype == torch.float32
    dlhs, drhs = torch.autograd.grad(o, (x_t, A_t), torch.from_numpy(dout).cuda())
    f64 = dict(out_dtype="float32", acc=np.float64)
    o_ref = oracle.gmm(lhs, rhs_in, gs, trans_rhs=trans_rhs, **f64)
    dlhs_ref, drhs_ref, _ = oracle.gmm_vjp(lhs, rhs_in, gs, dout, trans_rhs=trans_rhs, **f64)
    rows = np.arange(c["m"]) < target_m
    assert float(np.max(oracle.err_fn(util.to_np(o), o_ref, mask=rows))) < F32_EPS
    assert float(np.max(oracle.err_fn(util.to_np(dlhs), dlhs_ref, mask=rows))) < F32_EPS
    assert float(np.max(oracle.err_fn(util.to_np(drhs), drhs_ref, axis=(-1, -2), mask=gs != 0))) < F32_EPS
    assert not np.any(util.to_np(o)[target_m:]) and not np.any(util.to_np(dlhs)[target_m:])
    assert not np.any(util.to_np(drhs)[gs == 0])
    if not c["random_inputs"]:
        assert np.all(util.to_np(o)[:target_m] == c["k"])


@pytest.mark.parametrize("c", GRID[:16], ids=[util.case_id(c) for c in GRID[:16]])
def test_float32_trans_ragged_dot(c):
    print("f32 tgmm", c, flush=True)
    lhs, _, dout, gs, _ = _f32_case(c)
    out = rd.tgmm(torch.from_numpy(lhs).cuda(), torch.from_numpy(dout).cuda(), torch.from_numpy(gs))
    ref = oracle.tgmm(lhs, dout, gs, out_dtype="float32", acc=np.float64)
    assert float(np.max(oracle.err_fn(util.to_np(out), ref, axis=(-1, -2), mask=gs != 0))) < F32_TGMM_EPS
    assert not np.any(util.to_np(out)[gs == 0])


@pytest.mark.parametrize("shape", [(1030, 264, 392, 5), (515, 99, 131, 3), (600, 130, 262, 4), (2048, 128, 256, 2)],
                         ids=lambda s: "m%d_k%d_n%d_g%d" % s)
def test_float32_every_tile_shape(shape):
    """Each compiled float32 tile shape, forced through the plan, on shapes that take the 16-byte loads (all of k, n
    multiples of 4), the element loads (odd k, n) and a mix (k multiple of 2 only), against a float64 contraction."""
    from gpu_ragged_dot_amd import ops
    m, k, n, g = shape
    print("f32 tiles", shape, flush=True)
    rng = np.random.default_rng(m + k + n)
    lhs, rhs, dout = (rng.normal(size=s).astype(np.float32) for s in ((m, k), (g, k, n), (m, n)))
    gs = oracle.generate_group_sizes(11 + m, g, m - 37)
    rows = np.arange(m) < m - 37
    f64 = dict(out_dtype="float32", acc=np.float64)
    o_ref = oracle.gmm(lhs, rhs, gs, **f64)
    dlhs_ref = oracle.gmm(dout, rhs, gs, trans_rhs=True, **f64)
    drhs_ref = oracle.tgmm(lhs, dout, gs, **f64)
    x_t, A_t, d_t, gs_t = (torch.from_numpy(a).cuda() for a in (lhs, rhs, dout, gs))
    ids = [i for i, v in enumerate(_capi.variants()) if v.dtype == _capi.RD_DTYPE_F32]
    assert len(ids) >= 2
    for vid in ids:
        hp = (64, 64, 64)
        o = ops._gmm_fwd(x_t, A_t, gs_t, *hp, False, False, None, torch.float32, 512, plan=_capi.Plan(vid))
        dl = ops._gmm_fwd(d_t, A_t, gs_t, *hp, True, False, None, torch.float32, 512, plan=_capi.Plan(vid))
        dr = ops._tgmm_fwd(x_t, d_t, gs_t, *hp, False, None, torch.float32, 512, plan=_capi.Plan(vid))
        assert float(np.max(oracle.err_fn(util.to_np(o), o_ref, mask=rows))) < F32_EPS
        assert float(np.max(oracle.err_fn(util.to_np(dl), dlhs_ref, mask=rows))) < F32_EPS
        assert float(np.max(oracle.err_fn(util.to_np(dr), drhs_ref, axis=(-1, -2), mask=gs != 0))) < F32_TGMM_EPS
        assert not np.any(util.to_np(o)[m - 37:]) and not np.any(util.to_np(dl)[m - 37:])
        assert not np.any(util.to_np(dr)[gs == 0])


def test_streaming_default_with_all_rows_in_one_group():
    """The shape-only default picks the streaming kernel for m <= 4 g; the shape cannot see that all rows sit in one
    group, whose weights are then streamed once per 8 rows - every such pass a job of its own, spread over the
    work-groups."""
    print("streaming default, all rows in one group", flush=True)
    m, k, n, g = 256, 2048, 768, 128
    assert _capi.default_plan(_capi.OP_GMM, m, k, n, g).decode_nb == _capi.RD_DECODE_ROWS
    rng = np.random.default_rng(77)
    lhs = oracle.round_to(rng.standard_normal((m, k)).astype(np.float32), "bfloat16")
    rhs = oracle.round_to((rng.standard_normal((g, k, n)) / k ** 0.5).astype(np.float32), "bfloat16")
    for hot in (0, 77, g - 1):
        gs = np.zeros(g, np.int32)
        gs[hot] = m
        x, A, gsd = util.bf16_dev(lhs), util.bf16_dev(rhs), torch.from_numpy(gs).cuda()
        for trans_rhs in (False, True):
            Ad = A.mT.contiguous() if trans_rhs else A
            y = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
            assert _raw_gmm(x, Ad, gsd, y, trans_rhs=trans_rhs) == _capi.RD_OK, _capi.lib.rd_last_error()
            util.assert_close_rows(util.to_np(y), oracle.gmm(lhs, rhs, gs), m, util.BF16_EPS, f"hot={hot} t={trans_rhs}")


def test_stream_read_probe():
    """rd_probe_stream_read is a measurement aid, not part of the drop-in surface: it must run, store nothing, and
    refuse a source that is not 16-byte aligned."""
    print("stream read probe", flush=True)
    src = torch.arange(1 << 20, dtype=torch.int32, device="cuda")
    sink = torch.full((1,), 0x5a5a5a5a, dtype=torch.int32, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    for block in (16, 4096, 64 << 10, 3 << 20, 16 << 20):   # one thread's load .. more than the buffer
        rc = _capi.lib.rd_probe_stream_read(stream, src.data_ptr(), src.numel() * 4, block, sink.data_ptr())
        assert rc == _capi.RD_OK, _capi.lib.rd_last_error()
    assert _capi.lib.rd_probe_stream_read(stream, src.data_ptr(), src.numel() * 4 - 12, 4096, None) == _capi.RD_OK
    assert _capi.lib.rd_probe_stream_read(stream, src.data_ptr(), 0, 4096, None) == _capi.RD_OK
    torch.cuda.synchronize()
    assert int(sink.item()) == 0x5a5a5a5a
    assert torch.equal(src, torch.arange(1 << 20, dtype=torch.int32, device="cuda"))
    rc = _capi.lib.rd_probe_stream_read(stream, src.data_ptr() + 4, 4096, 4096, None)
    assert rc == _capi.RD_ERR_INVALID_ARGUMENT
    assert _capi.lib.rd_probe_stream_read(stream, src.data_ptr(), 4096, 8, None) == _capi.RD_ERR_INVALID_ARGUMENT
    assert _capi.lib.rd_probe_stream_read(stream, None, 4096, 4096, None) == _capi.RD_ERR_INVALID_ARGUMENT


# ---------------------------------------------------------------------------------------------------------------------
# every launch of a call goes to the caller's stream
# ---------------------------------------------------------------------------------------------------------------------

def test_calls_on_a_side_stream_wait_for_that_stream_only():
    """The inputs of each call are produced on a non-blocking side stream behind a long-running kernel, and the call is
    issued on that stream at once.  A launch of the library that went to another stream (a scheduling-map kernel, a
    finishing kernel, a zero fill) would run before its inputs exist and give a wrong result.  Covers the tile kernels
    with the interleaved block order and the K-split, tgmm with the group order, both streaming kernels of the default
    plan, and float32."""
    from gpu_ragged_dot_amd import ops
    print("side stream", flush=True)
    hp = dict(block_m=64, block_k=64, block_n=64, interpret=False, compute_dtype=None, acc_dtype=torch.float32, chunk_m=512)
    rng = np.random.default_rng(31)
    side = torch.cuda.Stream()

    def run(fn, host_inputs, dtype=torch.bfloat16):
        """fn(*device tensors) on the side stream; the device tensors start as zeros and are filled on that stream."""
        pinned = [torch.from_numpy(np.ascontiguousarray(a)).pin_memory() for a in host_inputs]
        devs = [torch.zeros(p.shape, dtype=(torch.int32 if p.dtype == torch.int32 else dtype), device="cuda") for p in pinned]
        torch.cuda.synchronize()
        with torch.cuda.stream(side):
            torch.cuda._sleep(20_000_000)           # at least several milliseconds during which nothing of this call may start
            for dvc, p in zip(devs, pinned):
                dvc.copy_(p.to(dvc.dtype) if p.dtype != torch.int32 else p, non_blocking=True)
            out = fn(*devs)
        side.synchronize()
        return util.to_np(out)

    # tile kernels: several rounds of tiles, long and short groups (interleaved block order)
    lens = list(rng.integers(1, 120, size=40)) + [0, 0, 700, 1300, 257, 530]
    rng.shuffle(lens)
    gs = np.array(lens, np.int32)
    m, k, n, g = int(gs.sum()) + 100, 72, 4096, len(lens)
    x = oracle.round_to(rng.standard_normal((m, k)).astype(np.float32), "bfloat16")
    w = oracle.round_to((rng.standard_normal((g, k, n)) / k ** 0.5).astype(np.float32), "bfloat16")
    got = run(lambda a, b, c: ops._gmm_fwd(a, b, c, **hp, trans_rhs=False), (x, w, gs))
    util.assert_close_rows(got, oracle.gmm(x, w, gs), int(gs.sum()), util.BF16_EPS, "side stream gmm")
    assert not np.any(got[int(gs.sum()):])

    # K-split of the last round (few tiles, long contraction), trans_rhs
    m, k, n, g = 900, 520, 7168, 5
    lhs, rhs, dout, gs, target_m = util.make_case(3, m, k, n, g, 0.9, True, scale_rhs=True)
    plan = _capi.Plan([v.id for v in _capi.variants() if v.name.decode() == "p256x256x32_w2x4_s4"][0], 2, 0, 2, 4)
    got = run(lambda a, b, c: ops._gmm_fwd(a, b, c, **hp, trans_rhs=True, plan=plan), (dout, rhs, gs))
    util.assert_close_rows(got, oracle.gmm(dout, rhs, gs, trans_rhs=True), target_m, util.BF16_EPS, "side stream dlhs")

    # tgmm with the groups visited by size class
    lens = [0, 1, 31, 64, 65, 128, 129, 300, 0, 7, 1100, 5, 40, 200, 95, 2]
    gs = np.array(lens, np.int32)
    m, k, n = int(gs.sum()) + 9, 264, 520
    x = oracle.round_to(rng.standard_normal((m, k)).astype(np.float32), "bfloat16")
    d = oracle.round_to(rng.standard_normal((m, n)).astype(np.float32), "bfloat16")
    plan = _capi.Plan(-1, 0, 0, 1)
    got = run(lambda a, b, c: ops._tgmm_fwd(a, b, c, **hp, plan=plan), (x, d, gs))
    util.assert_close_groups(got, oracle.tgmm(x, d, gs), gs != 0, util.TGMM_BF16_EPS, "side stream tgmm")
    assert not np.any(got[gs == 0])

    # the streaming kernels of the default plan: whole-row slices + finishing kernel, and the trans_rhs form
    m, k, n, g = 48, 1024, 512, 64
    lhs, rhs, _, gs, target_m = util.make_case(5, m, k, n, g, 0.9, True, scale_rhs=True)
    assert _capi.default_plan(_capi.OP_GMM, m, k, n, g).decode_nb == _capi.RD_DECODE_ROWS
    got = run(lambda a, b, c: ops._gmm_fwd(a, b, c, **hp, trans_rhs=False), (lhs, rhs, gs))
    util.assert_close_rows(got, oracle.gmm(lhs, rhs, gs), target_m, util.BF16_EPS, "side stream rows")
    assert not np.any(got[target_m:])
    rhs_t = np.ascontiguousarray(rhs.transpose(0, 2, 1))
    got = run(lambda a, b, c: ops._gmm_fwd(a, b, c, **hp, trans_rhs=True), (lhs, rhs_t, gs))
    util.assert_close_rows(got, oracle.gmm(lhs, rhs, gs), target_m, util.BF16_EPS, "side stream rows, weights transposed")

    # float32
    m, k, n, g = 300, 130, 77, 6
    rng2 = np.random.default_rng(8)
    x = rng2.standard_normal((m, k)).astype(np.float32)
    w = (rng2.standard_normal((g, k, n)) / k ** 0.5).astype(np.float32)
    gs = oracle.generate_group_sizes(4, g, 260)
    got = run(lambda a, b, c: ops._gmm_fwd(a, b, c, **hp, trans_rhs=False), (x, w, gs), dtype=torch.float32)
    util.assert_close_rows(got, oracle.gmm(x, w, gs, out_dtype="float32"), 260, 5e-4, "side stream float32")


# ---------------------------------------------------------------------------------------------------------------------
# HIP graph capture: no entry point reads device data on the host, so a captured step replays correctly
# ---------------------------------------------------------------------------------------------------------------------

def test_graph_capture_and_replay():
    """Forward + both backward products (tile kernels with the K-split, the streaming kernel, the routing kernels)
    captured once and replayed with new inputs in the same buffers: every replay must equal the eager result of the
    same inputs, with eager work and synchronisation in between."""
    from gpu_ragged_dot_amd import moe, ops
    print("graph capture", flush=True)
    hp = dict(block_m=64, block_k=64, block_n=64, interpret=False, compute_dtype=None, acc_dtype=torch.float32, chunk_m=512)
    m, k, n, g = 1500, 1096, 520, 6           # few tiles, long contraction: the K-split engages on the big tiles
    tokens, top_k = 750, 2
    gen = torch.Generator(device="cuda").manual_seed(0)

    def fresh():
        h = torch.randn((tokens, k), generator=gen, device="cuda").to(torch.bfloat16)
        A = (torch.randn((g, k, n), generator=gen, device="cuda") / k ** 0.5).to(torch.bfloat16)
        dout = torch.randn((m, n), generator=gen, device="cuda").to(torch.bfloat16)
        ids = torch.randint(0, g, (tokens, top_k), generator=gen, device="cuda", dtype=torch.int32)
        return h, A, dout, ids

    big = _capi.Plan([v.id for v in _capi.variants() if v.name.decode().startswith("q256")][0], 2, 0, 2)

    def step(h, A, dout, ids):
        r = moe.route(ids, g)
        x = moe._dispatch(h, r, None)
        y = ops._gmm_fwd(x, A, r.group_sizes, **hp, trans_rhs=False, plan=big)
        dx = ops._gmm_fwd(dout, A, r.group_sizes, **hp, trans_rhs=True, plan=big)
        dA = ops._tgmm_fwd(x, dout, r.group_sizes, **hp, plan=big)
        y_small = ops._gmm_fwd(x[:64].contiguous(), A, torch.clamp(r.group_sizes, max=10), **hp, trans_rhs=False,
                               plan=_capi.Plan(-1, 0, 64))
        out = moe._combine(y, r, None)
        return y, dx, dA, y_small, out

    static = [t.clone() for t in fresh()]
    step(*static)                              # warm-up: kernel attributes are set outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = step(*static)
    for _ in range(3):
        new = fresh()
        for dst, src in zip(static, new):
            dst.copy_(src)
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in captured]
        want = step(*new)                      # eager, on the default stream
        torch.cuda.synchronize()
        for a, b in zip(got, want):
            assert torch.equal(a, b)
