"""rd_gmm_noalloc: rd_gmm with the library's built-in per-device scratch buffer instead of a caller workspace.

Called through the C ABI and compared with rd_gmm on the same inputs and plan: same kernels, so bit-exact.  Two calls
in a row, the second on a smaller input, for the tile kernels and for the streaming (few rows per group) kernels, and
again on float32 and float8 arrays; sizes beyond the scratch buffer are refused with RD_ERR_WORKSPACE.
"""

import ctypes

import numpy as np
import pytest
import torch

from gpu_ragged_dot_amd import _capi
from oracle import ragged_dot_oracle as oracle
from tests import util

pytestmark = pytest.mark.gpu


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _plan_ref(plan):
    return ctypes.byref(plan) if plan is not None else None


def _run_both(x, A, gs_d, m, k, n, g, trans_rhs, dtype, plan, torch_dtype):
    outs = []
    for noalloc in (False, True):
        y = torch.full((m, n), float("nan"), dtype=torch_dtype, device="cuda")
        if noalloc:
            rc = _capi.lib.rd_gmm_noalloc(_stream(), x.data_ptr(), A.data_ptr(), gs_d.data_ptr(), y.data_ptr(), m, k, n, g,
                                          int(trans_rhs), dtype, _plan_ref(plan))
        else:
            ws = torch.empty(_capi.lib.rd_gmm_workspace_bytes(m, g, _plan_ref(plan)), dtype=torch.uint8, device="cuda")
            rc = _capi.lib.rd_gmm(_stream(), x.data_ptr(), A.data_ptr(), gs_d.data_ptr(), y.data_ptr(), m, k, n, g,
                                  int(trans_rhs), dtype, _plan_ref(plan), ws.data_ptr(), ws.numel())
        torch.cuda.synchronize()
        assert rc == 0, _capi.lib.rd_last_error()
        outs.append(y)
    return outs


@pytest.mark.parametrize("kind", ["tiles", "tiles_trans_rhs", "streaming_rows", "streaming_strips", "default_plan"])
def test_noalloc_matches_rd_gmm_on_two_calls_in_a_row(kind):
    assert _capi.lib.rd_gmm_noalloc_scratch_bytes() == 4 << 20
    big = [v.id for v in _capi.variants() if v.name.decode().startswith("w256")][0]
    if kind in ("tiles", "tiles_trans_rhs", "default_plan"):
        shapes = [(1500, 264, 520, 6, 0.9), (700, 136, 264, 3, 0.8)]   # the second call is the smaller one
        plan = None if kind == "default_plan" else _capi.Plan(big, 2, 0, 4, split_k=-1)
    else:
        shapes = [(48, 520, 264, 40, 1.0), (20, 136, 72, 9, 0.7)]
        plan = _capi.Plan(-1, 0, _capi.RD_DECODE_ROWS if kind == "streaming_rows" else 64, split_k=-1)
    trans_rhs = kind == "tiles_trans_rhs"
    for m, k, n, g, fill in shapes:
        print(f"noalloc {kind} m={m} k={k} n={n} g={g}", flush=True)
        lhs, rhs, _, gs, target_m = util.make_case(m + g, m, k, n, g, fill, True, scale_rhs=True)
        if kind.startswith("streaming"):
            gs = np.minimum(gs, 3).astype(np.int32)
            target_m = int(gs.sum())
        x = util.bf16_dev(lhs)
        A = util.bf16_dev(np.ascontiguousarray(np.swapaxes(rhs, 1, 2)) if trans_rhs else rhs)
        gs_d = torch.from_numpy(gs).cuda()
        ref, got = _run_both(x, A, gs_d, m, k, n, g, trans_rhs, _capi.RD_DTYPE_BF16, plan, torch.bfloat16)
        assert not torch.isnan(got).any()
        assert torch.equal(got, ref), "rd_gmm_noalloc differs from rd_gmm"
        util.assert_close_rows(util.to_np(got), oracle.gmm(lhs, rhs, gs), target_m, util.BF16_EPS, "y")
        assert not np.any(util.to_np(got)[target_m:])


def test_noalloc_float32_arrays():
    for dtype in (_capi.RD_DTYPE_F32, _capi.RD_DTYPE_F32_BF16):
        for m, k, n, g in ((600, 130, 262, 4), (300, 64, 136, 3)):
            rng = np.random.default_rng(m)
            lhs, rhs = rng.normal(size=(m, k)).astype(np.float32), rng.normal(size=(g, k, n)).astype(np.float32)
            gs = oracle.generate_group_sizes(m, g, m - 11)
            x, A, gs_d = torch.from_numpy(lhs).cuda(), torch.from_numpy(rhs).cuda(), torch.from_numpy(gs).cuda()
            ref, got = _run_both(x, A, gs_d, m, k, n, g, False, dtype, None, torch.float32)
            assert torch.equal(got, ref)


def test_noalloc_float8_operands():
    """float8 e4m3fn operands (bf16 out): the float8 matrix-core tiles in both weight layouts, and the streaming kernel
    for weights stored [g, n, k] (the default plan's choice for one row per group)."""
    for m, k, n, g, trans_rhs, streaming in ((600, 272, 528, 5, False, False), (300, 144, 272, 3, True, False),
                                             (40, 528, 264, 48, True, True), (12, 144, 72, 20, True, True)):
        print(f"noalloc float8 m={m} k={k} n={n} g={g} trans_rhs={trans_rhs}", flush=True)
        rng = np.random.default_rng(m)
        x8 = oracle.f32_to_float8_e4m3fn(rng.normal(size=(m, k)))
        A8 = oracle.f32_to_float8_e4m3fn(rng.normal(size=(g, k, n)) / np.sqrt(k))
        if streaming:
            gs = np.zeros(g, np.int32)
            gs[rng.choice(g, m - 3, replace=False)] = 1
            assert _capi.default_plan(_capi.OP_GMM_TRANS, m, k, n, g, _capi.RD_DTYPE_F8E4M3_BF16).decode_nb == _capi.RD_DECODE_ROWS
        else:
            gs = oracle.generate_group_sizes(m, g, m - 11)
        live = int(gs.sum())
        x = torch.from_numpy(x8).cuda().view(torch.float8_e4m3fn)
        A = torch.from_numpy(np.ascontiguousarray(np.swapaxes(A8, 1, 2)) if trans_rhs else A8).cuda().view(torch.float8_e4m3fn)
        ref, got = _run_both(x, A, torch.from_numpy(gs).cuda(), m, k, n, g, trans_rhs, _capi.RD_DTYPE_F8E4M3_BF16, None, torch.bfloat16)
        assert torch.equal(got, ref)
        y_ref = oracle.gmm(oracle.float8_e4m3fn_to_f32(x8), oracle.float8_e4m3fn_to_f32(A8), gs)
        util.assert_close_rows(util.to_np(got), y_ref, live, util.BF16_EPS, "y")
        assert not np.any(util.to_np(got)[live:])


def test_noalloc_refuses_what_does_not_fit():
    """A scheduling map beyond the 4 MiB scratch is refused with a status code before anything is launched."""
    m, g = 16 * 400_000, 4  # m / 16 + g row-tile slots: > 4 MiB of map
    plan = _capi.Plan(-1, 0, 0, 0, split_k=-1)
    assert _capi.lib.rd_gmm_workspace_bytes(m, g, ctypes.byref(plan)) > _capi.lib.rd_gmm_noalloc_scratch_bytes()
    one = torch.zeros(16, dtype=torch.bfloat16, device="cuda")
    gs = torch.zeros(g, dtype=torch.int32, device="cuda")
    rc = _capi.lib.rd_gmm_noalloc(_stream(), one.data_ptr(), one.data_ptr(), gs.data_ptr(), one.data_ptr(), m, 8, 8, g, 0,
                                  _capi.RD_DTYPE_BF16, None)
    assert rc == _capi.RD_ERR_WORKSPACE
    assert b"scratch" in _capi.lib.rd_last_error()
    torch.cuda.synchronize()
