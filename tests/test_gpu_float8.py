"""GPU parity for float8 e4m3fn operands (jax.lax.ragged_dot's float8 variant; the reference has no float8 path): the
HIP kernels multiply on the float8 matrix-core instruction where the row pitches are multiples of 16 bytes, and
otherwise widen the bytes to bf16 on their way into LDS and multiply on the bf16 matrix cores; fp32 accumulation and
bf16 output either way.  Everything goes through the C ABI (ctypes).  The oracle decodes the bytes by the format's definition and
computes in float64; since products of two e4m3 values are exact in fp32, what is left is the fp32 accumulation order
and the bf16 rounding of the result: the bf16 tolerances of the other parity tests apply unchanged."""

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
TGMM_EPS = 2e-2  # as the bf16 tgmm tests: rel-Frobenius per group slice


def _f8_dev(codes: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(codes)).cuda().view(torch.float8_e4m3fn)


def _case(seed, m, k, n, g, fill=0.9):
    rng = np.random.default_rng(seed)
    target_m = int(m * fill)
    gs = oracle.generate_group_sizes(seed, g, target_m)
    x8 = oracle.f32_to_float8_e4m3fn(rng.normal(size=(m, k)))
    A8 = oracle.f32_to_float8_e4m3fn(rng.normal(size=(g, k, n)) / np.sqrt(k))  # many subnormals among these
    d8 = oracle.f32_to_float8_e4m3fn(rng.normal(size=(m, n)))
    return x8, A8, d8, gs, target_m


def _f8_variants():
    return [v for v in _capi.variants() if v.dtype == _capi.RD_DTYPE_F8E4M3_BF16]


def test_every_code_passes_through_exactly():
    """x holds every finite code, A is a stack of identity matrices (1.0 = 0x38): y is x, exactly, as bf16."""
    k = 256
    codes = np.arange(256, dtype=np.uint8)
    finite = np.where((codes & 0x7F) == 0x7F, 0, codes)
    rng = np.random.default_rng(3)
    x8 = np.stack([np.roll(finite, s) for s in range(0, 96)] + [rng.permutation(finite) for _ in range(96)])  # [192, 256]
    eye = np.zeros((3, k, k), np.uint8)
    eye[:, np.arange(k), np.arange(k)] = 0x38
    gs = np.array([100, 0, 92], np.int32)
    want = oracle.float8_e4m3fn_to_f32(x8)
    for trans_rhs in (False, True):
        y = rd.gmm(_f8_dev(x8), _f8_dev(eye), torch.from_numpy(gs), trans_rhs=trans_rhs)
        assert y.dtype == torch.bfloat16
        assert np.array_equal(util.to_np(y), want), f"trans_rhs={trans_rhs}"
    # a NaN code poisons exactly its own row
    x8[5, 17] = 0x7F
    x8[150, 0] = 0xFF
    y = util.to_np(rd.gmm(_f8_dev(x8), _f8_dev(eye), torch.from_numpy(gs)))
    bad = np.isnan(y).any(axis=1)
    assert bad[5] and bad[150] and bad.sum() == 2
    assert np.isnan(y[5, 17]) and np.isnan(y[150, 0])


SHAPES = [(512, 256, 384, 4), (1030, 264, 392, 5), (515, 99, 131, 3), (300, 64, 64, 7), (2048, 512, 1024, 16), (64, 1024, 256, 32)]


@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "m%d_k%d_n%d_g%d" % s)
def test_float8_products_against_the_oracle(shape):
    """gmm (both layouts of A) and tgmm on ragged shapes with a zero tail and empty groups, default plan."""
    m, k, n, g = shape
    print("float8", shape, flush=True)
    x8, A8, d8, gs, target_m = _case(m + g, m, k, n, g)
    xf, Af, df = (oracle.float8_e4m3fn_to_f32(a) for a in (x8, A8, d8))
    gs_t = torch.from_numpy(gs)
    y_ref = oracle.gmm(xf, Af, gs)
    y = rd.gmm(_f8_dev(x8), _f8_dev(A8), gs_t)
    assert y.dtype == torch.bfloat16 and tuple(y.shape) == (m, n)
    util.assert_close_rows(util.to_np(y), y_ref, target_m, util.BF16_EPS, "gmm")
    assert not np.any(util.to_np(y)[target_m:])
    At8 = np.ascontiguousarray(np.swapaxes(A8, 1, 2))
    yt = rd.gmm(_f8_dev(x8), _f8_dev(At8), gs_t, trans_rhs=True)
    util.assert_close_rows(util.to_np(yt), y_ref, target_m, util.BF16_EPS, "gmm trans_rhs")
    dA_ref = oracle.tgmm(xf, df, gs)
    dA = rd.tgmm(_f8_dev(x8), _f8_dev(d8), gs_t)
    assert dA.dtype == torch.bfloat16 and tuple(dA.shape) == (g, k, n)
    util.assert_close_groups(util.to_np(dA), dA_ref, gs != 0, TGMM_EPS, "tgmm")
    assert not np.any(util.to_np(dA)[gs == 0])


@pytest.mark.parametrize("shape", [(1030, 264, 392, 5), (515, 99, 131, 3), (1300, 272, 520, 4), (700, 1040, 264, 9), (900, 528, 400, 6)],
                         ids=lambda s: "m%d_k%d_n%d_g%d" % s)
def test_float8_every_tile_shape(shape):
    """Each tile shape compiled for float8 operands, forced through the plan (the 8-byte-chunk ones only where the
    pitches allow), for gmm, gmm trans_rhs and tgmm; output NaN-poisoned first, rows below the output untouched."""
    m, k, n, g = shape
    x8, A8, d8, gs, target_m = _case(7 + m, m, k, n, g)
    xf, Af, df = (oracle.float8_e4m3fn_to_f32(a) for a in (x8, A8, d8))
    y_ref, dA_ref = oracle.gmm(xf, Af, gs), oracle.tgmm(xf, df, gs)
    x, A, d = _f8_dev(x8), _f8_dev(A8), _f8_dev(d8)
    At = _f8_dev(np.ascontiguousarray(np.swapaxes(A8, 1, 2)))
    gs_d = torch.from_numpy(gs).cuda()
    variants = _f8_variants()
    assert len(variants) >= 2 and any(not v.vec for v in variants)
    ran = 0
    guard = 32
    for v in variants:
        if v.vec and (k % 8 or n % 8):
            continue
        if v.direct_to_lds and k % 16:
            continue
        print("float8 tile", v.name.decode(), shape, flush=True)
        plan = _capi.Plan(v.id)
        ws = torch.empty(max(_capi.lib.rd_gmm_workspace_bytes(m, g, ctypes.byref(plan)), 256), dtype=torch.uint8, device="cuda")
        # the direct-to-LDS float8 shapes need 16-byte row pitches: n % 16 == 0 too when n is one (weights [g, k, n], tgmm)
        direct_needs_n16 = v.direct_to_lds and n % 16 != 0
        for trans_rhs, rhs in (((1, At),) if direct_needs_n16 else ((0, A), (1, At))):
            y = torch.full((m + guard, n), float("nan"), dtype=torch.bfloat16, device="cuda")
            rc = _capi.lib.rd_gmm(torch.cuda.current_stream().cuda_stream, x.data_ptr(), rhs.data_ptr(), gs_d.data_ptr(),
                                  y.data_ptr(), m, k, n, g, trans_rhs, _capi.RD_DTYPE_F8E4M3_BF16, ctypes.byref(plan),
                                  ws.data_ptr(), ws.numel())
            torch.cuda.synchronize()
            assert rc == 0, _capi.lib.rd_last_error()
            got = util.to_np(y)
            assert np.isnan(got[m:]).all() and not np.isnan(got[:m]).any()
            util.assert_close_rows(got[:m], y_ref, target_m, util.BF16_EPS, f"gmm {v.name.decode()} trans_rhs={trans_rhs}")
            assert not np.any(got[target_m:m])
        if direct_needs_n16:
            y = torch.empty((m, n), dtype=torch.bfloat16, device="cuda")
            rc = _capi.lib.rd_gmm(torch.cuda.current_stream().cuda_stream, x.data_ptr(), A.data_ptr(), gs_d.data_ptr(),
                                  y.data_ptr(), m, k, n, g, 0, _capi.RD_DTYPE_F8E4M3_BF16, ctypes.byref(plan),
                                  ws.data_ptr(), ws.numel())
            assert rc == _capi.RD_ERR_UNSUPPORTED  # refused by name, not mis-run
        if direct_needs_n16 or (v.direct_to_lds and v.tile_m % 256):  # (x^T as an operand: 256-row tiles only)
            with pytest.raises(_capi.RaggedDotError):
                ops._tgmm_fwd(x, d, gs_d, **HP, plan=plan)
            ran += 1
            continue
        dA = ops._tgmm_fwd(x, d, gs_d, **HP, plan=plan)
        util.assert_close_groups(util.to_np(dA), dA_ref, gs != 0, TGMM_EPS, f"tgmm {v.name.decode()}")
        assert not np.any(util.to_np(dA)[gs == 0])
        ran += 1
    assert ran >= 1


@pytest.mark.parametrize("trans_rhs", [0, 1], ids=["nn", "nt"])
@pytest.mark.parametrize("shape", [(900, 1104, 528, 5), (2100, 4112, 256, 3)], ids=lambda s: "m%d_k%d_n%d_g%d" % s)
def test_float8_k_split_of_last_round(shape, trans_rhs):
    """Few tiles and a long contraction on the float8 matrix-core shapes: the last round's tiles are cut along K over
    several work-groups.  Matches the oracle, agrees with the unsplit run up to fp32 summation order, overwrites every
    output element, and gives the same bits on a second call that reuses a workspace full of stale data."""
    m, k, n, g = shape
    x8, A8, _, gs, target_m = _case(11 + m, m, k, n, g)
    gs[1] = 0
    target_m = int(gs.sum())
    xf, Af = oracle.float8_e4m3fn_to_f32(x8), oracle.float8_e4m3fn_to_f32(A8)
    y_ref = oracle.gmm(xf, Af, gs)
    x = _f8_dev(x8)
    A = _f8_dev(np.ascontiguousarray(np.swapaxes(A8, 1, 2)) if trans_rhs else A8)
    gs_d = torch.from_numpy(gs).cuda()
    direct = [v for v in _f8_variants() if v.direct_to_lds]
    assert direct
    for v in direct:
        print("float8 k-split", v.name.decode(), shape, "trans_rhs", trans_rhs, flush=True)
        split, whole = _capi.Plan(v.id, 2, 0, 2, split_k=8), _capi.Plan(v.id, 2, 0, 2, split_k=-1)
        need = _capi.lib.rd_gmm_workspace_bytes(m, g, ctypes.byref(split))
        assert need > _capi.lib.rd_gmm_workspace_bytes(m, g, ctypes.byref(whole))
        ws = torch.empty(need, dtype=torch.uint8, device="cuda")
        ws.fill_(0xA5)
        outs = []
        for plan in (split, split, whole):
            y = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
            rc = _capi.lib.rd_gmm(torch.cuda.current_stream().cuda_stream, x.data_ptr(), A.data_ptr(), gs_d.data_ptr(),
                                  y.data_ptr(), m, k, n, g, trans_rhs, _capi.RD_DTYPE_F8E4M3_BF16, ctypes.byref(plan),
                                  ws.data_ptr(), ws.numel())
            torch.cuda.synchronize()
            assert rc == 0, _capi.lib.rd_last_error()
            outs.append(util.to_np(y))
        for y in outs:
            assert not np.isnan(y).any()
            util.assert_close_rows(y, y_ref, target_m, util.BF16_EPS, "y")
            assert not np.any(y[target_m:])
        assert np.array_equal(outs[0], outs[1])
        scale = np.abs(y_ref).max()
        assert np.abs(outs[0].astype(np.float32) - outs[2].astype(np.float32)).max() <= 2 ** -7 * scale


@pytest.mark.parametrize("trans_rhs", [0, 1], ids=["nn", "nt"])
@pytest.mark.parametrize("k,split_k", [(80, -1), (1104, -1), (4112, 8), (2048, 3)], ids=["k80", "k1104", "k4112-split8", "k2048-split3"])
def test_float8_short_group_row_tiles(k, split_k, trans_rhs):
    """Groups of 1..64 rows (the 64-row streaming routine inside the 256 x 256 float8 kernel), longer ones and the short
    last tile of a long group (tall routine) in one launch, contraction lengths that end inside a 128-deep and a 64-deep
    slab, with and without the K-split; twice, same bits."""
    vid = [v.id for v in _f8_variants() if v.direct_to_lds and v.tile_m == 256][0]
    gs = np.array([5, 64, 65, 128, 129, 0, 33, 100, 1, 256, 300, 257, 640], np.int32)
    m, n, g = int(gs.sum()) + 40, 528, gs.size
    print(f"float8 short tiles k={k} split_k={split_k} trans_rhs={trans_rhs}", flush=True)
    x8, A8, _, _, _ = _case(k, m, k, n, g, 1.0)
    target_m = int(gs.sum())
    y_ref = oracle.gmm(oracle.float8_e4m3fn_to_f32(x8), oracle.float8_e4m3fn_to_f32(A8), gs)
    x = _f8_dev(x8)
    A = _f8_dev(np.ascontiguousarray(np.swapaxes(A8, 1, 2)) if trans_rhs else A8)
    gs_d = torch.from_numpy(gs).cuda()
    plan = _capi.Plan(vid, 2, 0, 4, split_k=split_k)
    ws = torch.empty(_capi.lib.rd_gmm_workspace_bytes(m, g, ctypes.byref(plan)), dtype=torch.uint8, device="cuda")
    ws.fill_(0x3C)
    prev = None
    for _ in range(2):
        y = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
        rc = _capi.lib.rd_gmm(torch.cuda.current_stream().cuda_stream, x.data_ptr(), A.data_ptr(), gs_d.data_ptr(),
                              y.data_ptr(), m, k, n, g, trans_rhs, _capi.RD_DTYPE_F8E4M3_BF16, ctypes.byref(plan),
                              ws.data_ptr(), ws.numel())
        assert rc == 0, _capi.lib.rd_last_error()
        torch.cuda.synchronize()
        assert not torch.isnan(y).any()
        util.assert_close_rows(util.to_np(y), y_ref, target_m, util.BF16_EPS, "y")
        assert not torch.any(y[target_m:])
        assert prev is None or torch.equal(prev, y)
        prev = y


F8_STREAM_CASES = {
    "decode-shape": (2048, 768, None),
    "long-groups-tail": (528, 200, np.array([0, 11, 1, 0, 9, 5], np.int32)),
    "g600-sparse": (144, 72, None),
    "g300-two-rows": (272, 40, None),
    "wide-passes": (1040, 776, np.array([0, 1, 2, 3, 4, 5, 6, 7, 8, 0, 9, 12, 16, 17, 0, 3], np.int32)),
    "k8192": (8192, 64, np.array([2, 0, 1, 3], np.int32)),
    "n24": (2048, 24, np.array([1, 0, 4, 2, 0, 0, 1, 1], np.int32)),
    "k16": (16, 136, np.array([3, 0, 1], np.int32)),
}


@pytest.mark.parametrize("case", list(F8_STREAM_CASES))
def test_float8_streaming_kernel_trans_rhs(case):
    """float8 weights stored [g, n, k] and a few rows per group: the streaming kernel that cuts every expert's weight
    rows into blocks along n, widens the bytes to bf16 in registers and writes y in one launch.  By name and by the
    default plan; 4 and 8 rows per pass, groups that need several passes, empty groups, a zero tail, contraction lengths
    that are not a whole number of 1024-element positions, more non-empty groups than work-groups, fewer output columns
    than pieces.  Its sums are those of the tile kernels up to fp32 addition order."""
    print(f"float8 streaming kernel, trans_rhs, {case}", flush=True)
    rng = np.random.default_rng(len(case))
    k, n, gs = F8_STREAM_CASES[case]
    if case == "decode-shape":
        gs = np.zeros(128, np.int32)
        np.add.at(gs, rng.integers(0, 128, 64), 1)
    elif gs is None:
        g, active, rows_each = (600, 40, 1) if case == "g600-sparse" else (300, 299, 2)
        gs = np.zeros(g, np.int32)
        gs[rng.choice(g, active, replace=False)] = rows_each
    g, m = len(gs), int(gs.sum()) + 5
    x8 = oracle.f32_to_float8_e4m3fn(rng.normal(size=(m, k)))
    A8 = oracle.f32_to_float8_e4m3fn(rng.normal(size=(g, k, n)) / np.sqrt(k))
    y_ref = oracle.gmm(oracle.float8_e4m3fn_to_f32(x8), oracle.float8_e4m3fn_to_f32(A8), gs)
    At = _f8_dev(np.ascontiguousarray(np.swapaxes(A8, 1, 2)))
    x, gs_t = _f8_dev(x8), torch.from_numpy(gs)
    live = int(gs.sum())
    if case == "decode-shape":
        assert _capi.default_plan(_capi.OP_GMM_TRANS, m, k, n, g, _capi.RD_DTYPE_F8E4M3_BF16).decode_nb == _capi.RD_DECODE_ROWS
    for plan in (_capi.Plan(-1, 0, _capi.RD_DECODE_ROWS), None):
        y = util.to_np(ops._gmm_fwd(x, At, gs_t, **HP, trans_rhs=True, plan=plan))
        util.assert_close_rows(y, y_ref, live, util.BF16_EPS, f"float8 trans_rhs streaming kernel plan={plan}")
        assert not np.any(y[live:])
    # forced onto a tile kernel: the same sums
    tile = [v.id for v in _f8_variants() if not v.vec][0]
    y_tile = util.to_np(ops._gmm_fwd(x, At, gs_t, **HP, trans_rhs=True, plan=_capi.Plan(tile)))
    scale = max(np.abs(y_ref).max(), 1e-6)
    assert np.abs(y.astype(np.float32) - y_tile.astype(np.float32)).max() <= 2 ** -6 * scale


def test_float8_streaming_kernel_limits():
    """What the float8 streaming kernel does not serve is refused by name and left to the tile kernels by default:
    weights stored [g, k, n], a contraction too long to stage, a pitch that is not a multiple of 16."""
    rng = np.random.default_rng(2)
    gs = np.array([1, 2], np.int32)
    for k, n, trans_rhs in ((512, 64, False), (8208, 16, True), (520, 64, True)):
        x8 = oracle.f32_to_float8_e4m3fn(rng.normal(size=(3, k)))
        A8 = oracle.f32_to_float8_e4m3fn(rng.normal(size=(2, k, n)) / np.sqrt(k))
        y_ref = oracle.gmm(oracle.float8_e4m3fn_to_f32(x8), oracle.float8_e4m3fn_to_f32(A8), gs)
        A = _f8_dev(np.ascontiguousarray(np.swapaxes(A8, 1, 2)) if trans_rhs else A8)
        args = (_f8_dev(x8), A, torch.from_numpy(gs))
        print(f"float8 streaming limits k={k} n={n} trans_rhs={trans_rhs}", flush=True)
        for nb in (_capi.RD_DECODE_ROWS, 64):
            if not trans_rhs:  # [g, k, n]: a streaming plan is dropped, as for every element type without those kernels
                y = ops._gmm_fwd(*args, **HP, trans_rhs=False, plan=_capi.Plan(-1, 0, nb))
                util.assert_close_rows(util.to_np(y), y_ref, 3, util.BF16_EPS, "dropped plan")
                continue
            with pytest.raises(_capi.RaggedDotError):
                ops._gmm_fwd(*args, **HP, trans_rhs=trans_rhs, plan=_capi.Plan(-1, 0, nb))
        util.assert_close_rows(util.to_np(ops._gmm_fwd(*args, **HP, trans_rhs=trans_rhs)), y_ref, 3, util.BF16_EPS, "default")


def test_float8_is_forward_only_and_rejects_mixed_operands():
    x8, A8, _, gs, _ = _case(1, 128, 64, 64, 2)
    x, A = _f8_dev(x8), _f8_dev(A8)
    gs_t = torch.from_numpy(gs)
    with pytest.raises(TypeError):
        rd.gmm(x, A.to(torch.bfloat16), gs_t)
    with pytest.raises(NotImplementedError):
        rd.gmm(x, A, gs_t, compute_dtype=torch.float16)
    try:
        xr = x.clone().requires_grad_(True)
    except RuntimeError:
        return  # this torch does not let a float8 tensor require a gradient at all
    with pytest.raises(NotImplementedError):
        rd.gmm(xr, A, gs_t)
    # a bf16 variant forced on float8 operands is refused with a status code
    bf16 = [v.id for v in _capi.variants() if v.dtype == _capi.RD_DTYPE_BF16][0]
    with pytest.raises(_capi.RaggedDotError):
        ops._gmm_fwd(x, A, gs_t, **HP, trans_rhs=False, plan=_capi.Plan(bf16))
