"""Operands with more than 2^31 elements (element offsets that do not fit a 32-bit integer): tall x / y / dout with a
small stack of weights, and a stack of weights / a weights cotangent beyond 2^31 elements with few rows.  Sampled rows
and slices are compared with float64 products of the same rows on the host and with torch's fp32 matmuls on the
device; samples sit on both sides of element 2^31, at the ends of groups and in the zero tail."""

import numpy as np
import pytest
import torch

import gpu_ragged_dot_amd as rd
from tests import util

pytestmark = pytest.mark.gpu


def _rows_f64(x_rows, W):
    return util.to_np(x_rows).astype(np.float64) @ util.to_np(W).astype(np.float64)


def test_tall_activations_beyond_2_31_elements():
    m, k, n, g = 1_200_000, 2048, 2048, 3
    assert m * k > 2 ** 31 and m * n > 2 ** 31
    print("big index: tall", m, k, n, flush=True)
    gen = torch.Generator(device="cuda").manual_seed(4)
    x = torch.randn((m, k), generator=gen, device="cuda", dtype=torch.bfloat16)
    A = (torch.randn((g, k, n), generator=gen, device="cuda") / k ** 0.5).to(torch.bfloat16)
    gs = np.array([500_000, 0, 650_000], np.int32)  # 50 000 rows of tail
    gs_t = torch.from_numpy(gs)
    off = np.concatenate([[0], np.cumsum(gs)])
    edge = 2 ** 31 // k  # the row whose first element has offset 2^31
    sample = {0: [0, 1, 499_999], 2: [500_000, edge - 1, edge, edge + 1, 1_149_999]}

    y = rd.gmm(x, A, gs_t)
    At = A.transpose(1, 2).contiguous()
    yt = rd.gmm(x, At, gs_t, trans_rhs=True)
    torch.cuda.synchronize()
    for gi, rows in sample.items():
        rt = torch.tensor(rows, device="cuda")
        ref = _rows_f64(x[rt], A[gi])
        util.assert_close_rows(util.to_np(y[rt]).astype(np.float64), ref, len(rows), util.BF16_EPS, f"y g{gi}")
        util.assert_close_rows(util.to_np(yt[rt]).astype(np.float64), ref, len(rows), util.BF16_EPS, f"y trans_rhs g{gi}")
    assert not torch.any(y[int(off[-1]):]).item() and not torch.any(yt[int(off[-1]):]).item()
    assert torch.any(y[int(off[-1]) - 1]).item()
    # a stretch of rows across the 2^31 boundary against torch's fp32 matmul
    band = slice(edge - 300, edge + 300)
    ref_band = (x[band].float() @ A[2].float()).to(torch.bfloat16)
    util.assert_close_rows(util.to_np(y[band]), util.to_np(ref_band), 600, util.BF16_EPS, "y across 2^31")
    del yt, ref_band

    # tgmm over the same tall operands (y doubles as dout): contraction over 500 000 and 650 000 rows
    dA = rd.tgmm(x, y, gs_t)
    torch.cuda.synchronize()
    assert not torch.any(dA[1]).item()
    for gi in (0, 2):
        lo, hi = int(off[gi]), int(off[gi + 1])
        ref = torch.zeros((k, n), dtype=torch.float32, device="cuda")
        for s in range(lo, hi, 65536):  # fp32 partial products, summed in fp32
            e = min(hi, s + 65536)
            ref += x[s:e].float().T @ y[s:e].float()
        util.assert_close_groups(util.to_np(dA[gi])[None], util.to_np(ref)[None], np.array([True]), util.TGMM_BF16_EPS * 2, f"drhs g{gi}")


def test_stacked_weights_beyond_2_31_elements():
    m, k, n, g = 4096, 8192, 8192, 40
    assert g * k * n > 2 ** 31
    print("big index: weights", m, k, n, g, flush=True)
    gen = torch.Generator(device="cuda").manual_seed(9)
    x = torch.randn((m, k), generator=gen, device="cuda", dtype=torch.bfloat16)
    dout = torch.randn((m, n), generator=gen, device="cuda", dtype=torch.bfloat16)
    A = torch.empty((g, k, n), device="cuda", dtype=torch.bfloat16)
    for i in range(g):
        A[i] = (torch.randn((k, n), generator=gen, device="cuda") / k ** 0.5).to(torch.bfloat16)
    gs = np.full(g, 100, np.int32)
    gs[[3, 31, 35]] = [0, 196, 0]  # 3896 rows, 200 of tail; group 31 straddles element 2^31 of A, 32.. lie beyond it
    gs_t = torch.from_numpy(gs)
    off = np.concatenate([[0], np.cumsum(gs)])
    assert 31 * k * n < 2 ** 31 <= 32 * k * n

    y = rd.gmm(x, A, gs_t)
    dx = rd.gmm(dout, A, gs_t, trans_rhs=True)
    dA = rd.tgmm(x, dout, gs_t)
    torch.cuda.synchronize()
    for gi in (0, 31, 32, 39):
        lo, hi = int(off[gi]), int(off[gi + 1])
        rows = [lo, (lo + hi) // 2, hi - 1]
        rt = torch.tensor(rows, device="cuda")
        util.assert_close_rows(util.to_np(y[rt]).astype(np.float64), _rows_f64(x[rt], A[gi]), 3, util.BF16_EPS, f"y g{gi}")
        util.assert_close_rows(util.to_np(dx[rt]).astype(np.float64), _rows_f64(dout[rt], A[gi].T), 3, util.BF16_EPS, f"dlhs g{gi}")
        ref = (x[lo:hi].float().T @ dout[lo:hi].float())
        util.assert_close_groups(util.to_np(dA[gi])[None], util.to_np(ref)[None], np.array([True]), util.TGMM_BF16_EPS, f"drhs g{gi}")
    assert not torch.any(y[int(off[-1]):]).item() and not torch.any(dx[int(off[-1]):]).item()
    assert not torch.any(dA[3]).item() and not torch.any(dA[35]).item()
