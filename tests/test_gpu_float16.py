"""float16 arrays (RD_DTYPE_F16): the reference takes whatever element type its arrays have (gpu_ragged_dot.py:116-119,
210, 324); here float16 runs on the float16 matrix-core instruction with fp32 accumulation and float16 out.
Oracle: the float32 contraction of the float16 values, rounded once to float16 (numpy's conversion, nearest even;
pinned in tests/test_oracle.py).  Tolerances: the reference's bf16 ones (tests.py:127,144,168,183) divided by five -
float16 carries three more mantissa bits than bfloat16."""

import numpy as np
import pytest
import torch

import gpu_ragged_dot_amd as rd
from gpu_ragged_dot_amd import _capi
from oracle import ragged_dot_oracle as oracle
from tests import util

pytestmark = pytest.mark.gpu

F16_EPS = util.BF16_EPS / 5
F16_TGMM_EPS = util.TGMM_BF16_EPS / 2
GRID = util.reference_grid(24, seed=3)


def _dev(a):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).cuda().to(torch.float16)


def _case(c, scale=True):
    rng = np.random.default_rng(c["seed"] * 131 + c["m"] + 3 * c["k"] + 5 * c["n"] + c["g"])
    m, k, n, g = c["m"], c["k"], c["n"], c["g"]
    if c["random_inputs"]:
        lhs = rng.normal(size=(m, k)).astype(np.float32)
        rhs = (rng.normal(size=(g, k, n)) / (np.sqrt(k) if scale else 1.0)).astype(np.float32)
        dout = rng.normal(size=(m, n)).astype(np.float32)
    else:
        lhs, rhs, dout = (np.ones(s, np.float32) for s in ((m, k), (g, k, n), (m, n)))
    lhs, rhs, dout = (oracle.round_to(a, "float16") for a in (lhs, rhs, dout))
    target_m = max(min(round(m * c["fill_in"]), m), 0)
    gs = oracle.generate_group_sizes(c["seed"] + 7 * g + target_m, g, target_m)
    return lhs, rhs, dout, gs, target_m


@pytest.mark.parametrize("trans_rhs", [False, True], ids=["A", "At"])
@pytest.mark.parametrize("c", GRID[:16], ids=[util.case_id(c) for c in GRID[:16]])
def test_float16_forward_and_vjp(c, trans_rhs):
    print("f16", c, "trans_rhs", trans_rhs, flush=True)
    lhs, rhs, dout, gs, target_m = _case(c)
    rhs_in = np.ascontiguousarray(np.swapaxes(rhs, 1, 2)) if trans_rhs else rhs
    x_t, A_t = _dev(lhs).requires_grad_(True), _dev(rhs_in).requires_grad_(True)
    o = rd.gmm(x_t, A_t, torch.from_numpy(gs), block_m=c["block_m"], block_k=c["block_k"], block_n=c["block_n"],
               chunk_m=c["chunk_m"], trans_rhs=trans_rhs)
    assert o.dtype == torch.float16
    dlhs, drhs = torch.autograd.grad(o, (x_t, A_t), _dev(dout))
    assert dlhs.dtype == torch.float16 and drhs.dtype == torch.float16
    f16 = dict(out_dtype="float16")
    o_ref = oracle.gmm(lhs, rhs_in, gs, trans_rhs=trans_rhs, **f16)
    dlhs_ref, drhs_ref, _ = oracle.gmm_vjp(lhs, rhs_in, gs, dout, trans_rhs=trans_rhs, **f16)
    util.assert_close_rows(util.to_np(o), o_ref, target_m, F16_EPS, "f16 gmm")
    util.assert_close_rows(util.to_np(dlhs), dlhs_ref, target_m, F16_EPS, "f16 dlhs")
    if np.any(gs != 0):
        util.assert_close_groups(util.to_np(drhs), drhs_ref, gs != 0, F16_TGMM_EPS, "f16 drhs")
    assert not np.any(util.to_np(o)[target_m:]) and not np.any(util.to_np(dlhs)[target_m:])
    assert not np.any(util.to_np(drhs)[gs == 0])
    if not c["random_inputs"]:
        assert np.all(util.to_np(o)[:target_m] == c["k"])   # k <= 512 is a float16 value


@pytest.mark.parametrize("c", GRID[16:24], ids=[util.case_id(c) for c in GRID[16:24]])
def test_float16_trans_ragged_dot(c):
    print("f16 tgmm", c, flush=True)
    lhs, _, dout, gs, _ = _case(c)
    out = rd.tgmm(_dev(lhs), _dev(dout), torch.from_numpy(gs))
    assert out.dtype == torch.float16
    ref = oracle.tgmm(lhs, dout, gs, out_dtype="float16")
    if np.any(gs != 0):
        util.assert_close_groups(util.to_np(out), ref, gs != 0, F16_TGMM_EPS, "f16 tgmm")
    assert not np.any(util.to_np(out)[gs == 0])


@pytest.mark.parametrize("shape", [(1030, 264, 392, 5), (515, 99, 131, 3), (600, 130, 262, 4), (2048, 128, 256, 2)],
                         ids=lambda s: "m%d_k%d_n%d_g%d" % s)
def test_float16_every_tile_shape(shape):
    """Each compiled float16 tile shape, forced through the plan, on 16-byte pitches, odd pitches and a mix; a shape
    asked for pitches it cannot serve must refuse."""
    from gpu_ragged_dot_amd import ops
    m, k, n, g = shape
    print("f16 tiles", shape, flush=True)
    rng = np.random.default_rng(m + k + n)
    lhs = oracle.round_to(rng.normal(size=(m, k)).astype(np.float32), "float16")
    rhs = oracle.round_to((rng.normal(size=(g, k, n)) / np.sqrt(k)).astype(np.float32), "float16")
    dout = oracle.round_to(rng.normal(size=(m, n)).astype(np.float32), "float16")
    gs = oracle.generate_group_sizes(11 + m, g, m - 37)
    o_ref = oracle.gmm(lhs, rhs, gs, out_dtype="float16")
    dlhs_ref = oracle.gmm(dout, rhs, gs, trans_rhs=True, out_dtype="float16")
    drhs_ref = oracle.tgmm(lhs, dout, gs, out_dtype="float16")
    x_t, A_t, d_t, gs_t = _dev(lhs), _dev(rhs), _dev(dout), torch.from_numpy(gs).cuda()
    variants = [v for v in _capi.variants() if v.dtype == _capi.RD_DTYPE_F16]
    assert len(variants) >= 3 and any(not v.vec for v in variants)
    hp = dict(block_m=64, block_k=64, block_n=64, interpret=False, compute_dtype=None, acc_dtype=torch.float32, chunk_m=512)
    aligned = k % 8 == 0 and n % 8 == 0
    served = 0
    for v in variants:
        plan = _capi.Plan(v.id)
        if v.vec and not aligned:
            with pytest.raises(_capi.RaggedDotError) as e:
                ops._gmm_fwd(x_t, A_t, gs_t, **hp, trans_rhs=False, plan=plan)
            assert e.value.status == _capi.RD_ERR_UNSUPPORTED
            continue
        o = ops._gmm_fwd(x_t, A_t, gs_t, **hp, trans_rhs=False, plan=plan)
        dl = ops._gmm_fwd(d_t, A_t, gs_t, **hp, trans_rhs=True, plan=plan)
        dr = ops._tgmm_fwd(x_t, d_t, gs_t, **hp, plan=plan)
        util.assert_close_rows(util.to_np(o), o_ref, m - 37, F16_EPS, v.name.decode())
        util.assert_close_rows(util.to_np(dl), dlhs_ref, m - 37, F16_EPS, v.name.decode())
        util.assert_close_groups(util.to_np(dr), drhs_ref, gs != 0, F16_TGMM_EPS, v.name.decode())
        assert not np.any(util.to_np(o)[m - 37:]) and not np.any(util.to_np(dl)[m - 37:])
        assert not np.any(util.to_np(dr)[gs == 0])
        served += 1
    assert served >= 1


def test_float16_extremes_and_types():
    """Values at the ends of the float16 range go through exactly (an identity product), a product that overflows
    float16 becomes infinity as the rounding of its fp32 value does, and mixed element types are refused."""
    k = n = 64
    vals = np.array([65504.0, -65504.0, 2.0 ** -24, -2.0 ** -24, 2.0 ** -14, 1.0 + 2.0 ** -10, 0.0, -0.0], np.float32)
    x = np.zeros((len(vals), k), np.float32)
    x[:, 5] = vals
    eye = np.eye(k, n, dtype=np.float32)[None]
    gs = np.array([len(vals)], np.int32)
    y = util.to_np(rd.gmm(_dev(x), _dev(eye), torch.from_numpy(gs)))
    assert np.array_equal(y[:, 5], vals) and not np.any(np.delete(y, 5, axis=1))
    two = 2.0 * eye
    y = util.to_np(rd.gmm(_dev(x), _dev(two), torch.from_numpy(gs)))
    assert np.isposinf(y[0, 5]) and np.isneginf(y[1, 5]) and y[2, 5] == 2.0 ** -23
    with pytest.raises(TypeError):
        rd.gmm(_dev(x), torch.from_numpy(eye).cuda().to(torch.bfloat16), torch.from_numpy(gs))


def test_float16_default_plan_on_a_larger_shape():
    """The library's own choice (no plan) on a shape with a few hundred tiles, ragged groups and a zero tail."""
    m, k, n, g = 3000, 520, 1032, 7
    rng = np.random.default_rng(5)
    lhs = oracle.round_to(rng.normal(size=(m, k)).astype(np.float32), "float16")
    rhs = oracle.round_to((rng.normal(size=(g, k, n)) / np.sqrt(k)).astype(np.float32), "float16")
    dout = oracle.round_to(rng.normal(size=(m, n)).astype(np.float32), "float16")
    gs = oracle.generate_group_sizes(3, g, 2800)
    assert _capi.default_plan(_capi.OP_GMM, m, k, n, g, _capi.RD_DTYPE_F16).variant >= 0
    o = util.to_np(rd.gmm(_dev(lhs), _dev(rhs), torch.from_numpy(gs)))
    util.assert_close_rows(o, oracle.gmm(lhs, rhs, gs, out_dtype="float16"), 2800, F16_EPS, "f16 default gmm")
    assert not np.any(o[2800:])
    dr = util.to_np(rd.tgmm(_dev(lhs), _dev(dout), torch.from_numpy(gs)))
    util.assert_close_groups(dr, oracle.tgmm(lhs, dout, gs, out_dtype="float16"), gs != 0, F16_TGMM_EPS, "f16 default tgmm")


@pytest.mark.parametrize("trans_rhs,k", [(False, 264), (True, 520), (True, 1800)], ids=["A_k264", "At_k520", "At_k1800"])
def test_float16_four_wave_core(trans_rhs, k):
    """The 256 x 256 direct-to-LDS core compiled with the float16 instruction (the default for float16 where bf16 arrays
    would take a 256 x 256 core): groups of every length class - the streaming routines for up to 64 and up to 128 rows
    run inside the same launch - a zero tail, partial column tiles, the contraction on both sides of the length at which
    trans_rhs moves to the register-staged form, the K-split forced, and tgmm."""
    from gpu_ragged_dot_amd import ops
    print("f16 four-wave core", trans_rhs, k, flush=True)
    lens = [0, 1, 31, 64, 65, 128, 129, 300, 0, 7, 700, 5, 40, 257, 95, 2, 513]
    gs = np.array(lens, np.int32)
    g, n = len(lens), 776
    m = int(gs.sum()) + 50
    rng = np.random.default_rng(k + int(trans_rhs))
    lhs = oracle.round_to(rng.normal(size=(m, k)).astype(np.float32), "float16")
    rhs = oracle.round_to((rng.normal(size=(g, k, n)) / np.sqrt(k)).astype(np.float32), "float16")
    dout = oracle.round_to(rng.normal(size=(m, n)).astype(np.float32), "float16")
    vid = [v.id for v in _capi.variants() if v.name.decode() == "hw256x256x32_w2x2_s5"][0]
    hp = dict(block_m=64, block_k=64, block_n=64, interpret=False, compute_dtype=None, acc_dtype=torch.float32, chunk_m=512)
    rhs_in = np.ascontiguousarray(np.swapaxes(rhs, 1, 2)) if trans_rhs else rhs
    ref = oracle.gmm(lhs, rhs_in, gs, trans_rhs=trans_rhs, out_dtype="float16")
    outs = []
    for split_k in (-1, 0, 2):
        plan = _capi.Plan(vid, 2, 0, 2, split_k)
        o = ops._gmm_fwd(_dev(lhs), _dev(rhs_in), torch.from_numpy(gs), **hp, trans_rhs=trans_rhs, plan=plan)
        assert o.dtype == torch.float16
        util.assert_close_rows(util.to_np(o), ref, int(gs.sum()), F16_EPS, f"split_k={split_k}")
        assert not np.any(util.to_np(o)[int(gs.sum()):])
        outs.append(o)
    assert torch.equal(outs[0].view(torch.int16), outs[1].view(torch.int16))   # (k < 6400: the default does not split)
    dr = ops._tgmm_fwd(_dev(lhs), _dev(dout), torch.from_numpy(gs), **hp, plan=_capi.Plan(vid, 4, 0, 1))
    util.assert_close_groups(util.to_np(dr), oracle.tgmm(lhs, dout, gs, out_dtype="float16"), gs != 0, F16_TGMM_EPS, "tgmm")
    assert not np.any(util.to_np(dr)[gs == 0])


def test_float16_default_is_the_four_wave_core_on_large_shapes():
    vs = {v.id: v.name.decode() for v in _capi.variants()}
    for op, shape in ((_capi.OP_GMM, (16384, 4096, 14336, 8)), (_capi.OP_GMM_TRANS, (16384, 14336, 4096, 8)),
                      (_capi.OP_TGMM, (16384, 4096, 14336, 8)), (_capi.OP_GMM, (32768, 7168, 2048, 256))):
        assert vs[_capi.default_plan(op, *shape, _capi.RD_DTYPE_F16).variant] == "hw256x256x32_w2x2_s5"
    small = _capi.default_plan(_capi.OP_GMM, 300, 128, 256, 4, _capi.RD_DTYPE_F16)
    assert vs[small.variant].startswith("h") and small.decode_nb == 0
    assert _capi.default_plan(_capi.OP_GMM, 64, 2048, 768, 128, _capi.RD_DTYPE_F16).decode_nb == _capi.RD_DECODE_ROWS
    assert _capi.default_plan(_capi.OP_GMM_TRANS, 64, 2048, 768, 128, _capi.RD_DTYPE_F16).decode_nb == _capi.RD_DECODE_ROWS


@pytest.mark.parametrize("m,hot", [(48, None), (200, None), (256, 5)], ids=["m48", "m200", "m256_one_group"])
def test_float16_streaming_kernels(m, hot):
    """A few rows per group: the streaming kernels in float16 - whole-row slices with 4 and with 8 rows per pass and
    their finishing kernel, the form for weights stored [g, n, k], the column-strip kernel at its three widths - under
    the default plan and forced, with empty groups, a zero tail, and all rows piled into one group."""
    from gpu_ragged_dot_amd import ops
    print("f16 streaming", m, hot, flush=True)
    k, n, g = 1024, 512, 64
    rng = np.random.default_rng(m)
    if hot is None:
        gs = oracle.generate_group_sizes(m, g, m - 5)
        gs[rng.random(g) < 0.3] = 0
    else:
        gs = np.zeros(g, np.int32)
        gs[hot] = m - 5
    live = int(gs.sum())
    lhs = oracle.round_to(rng.normal(size=(m, k)).astype(np.float32), "float16")
    rhs = oracle.round_to((rng.normal(size=(g, k, n)) / np.sqrt(k)).astype(np.float32), "float16")
    ref = oracle.gmm(lhs, rhs, gs, out_dtype="float16")
    hp = dict(block_m=64, block_k=64, block_n=64, interpret=False, compute_dtype=None, acc_dtype=torch.float32, chunk_m=512)
    x_t, A_t, gs_t = _dev(lhs), _dev(rhs), torch.from_numpy(gs)
    At_t = A_t.mT.contiguous()
    assert _capi.default_plan(_capi.OP_GMM, m, k, n, g, _capi.RD_DTYPE_F16).decode_nb == _capi.RD_DECODE_ROWS
    plans = [None, _capi.Plan(-1, 0, _capi.RD_DECODE_ROWS), _capi.Plan(-1, 0, 32), _capi.Plan(-1, 0, 64), _capi.Plan(-1, 0, 128)]
    for plan in plans:
        o = ops._gmm_fwd(x_t, A_t, gs_t, **hp, trans_rhs=False, plan=plan)
        assert o.dtype == torch.float16
        util.assert_close_rows(util.to_np(o), ref, live, F16_EPS, f"plan {plan}")
        assert not np.any(util.to_np(o)[live:])
    for plan in (None, _capi.Plan(-1, 0, _capi.RD_DECODE_ROWS)):
        o = ops._gmm_fwd(x_t, At_t, gs_t, **hp, trans_rhs=True, plan=plan)
        util.assert_close_rows(util.to_np(o), ref, live, F16_EPS, f"weights transposed, plan {plan}")
        assert not np.any(util.to_np(o)[live:])
