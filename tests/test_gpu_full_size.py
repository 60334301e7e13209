"""Parity at the benchmark's full sizes (Mixtral- and DeepSeek-V3-shaped forward + VJP).

The numpy oracle cannot multiply these in seconds, so each product is checked (a) on sampled rows / groups against the
oracle, (b) on the same samples against fp32 matmuls by torch (hipBLASLt: code independent of these kernels), and
(c) through size-independent properties: empty groups exactly zero, adjoint identity <dout, y> = <dlhs, x> = <drhs, A>.
"""

import numpy as np
import pytest
import torch

import gpu_ragged_dot_amd as rd
from gpu_ragged_dot_amd import workloads
from oracle import ragged_dot_oracle as oracle
from tests import util

pytestmark = pytest.mark.gpu


def _sample_groups(gs):
    nz = np.flatnonzero(gs > 0)
    picks = {int(nz[0]), int(nz[-1]), int(nz[np.argmax(gs[nz])]), int(nz[np.argmin(gs[nz])]), int(nz[len(nz) // 2])}
    return sorted(picks)


@pytest.mark.parametrize("name", ["mixtral_fwd_bwd", "deepseek_fwd_bwd"])
def test_full_size_forward_and_vjp(name):
    print("full size", name, flush=True)
    x, A, dout, gs_t = workloads.make_inputs(name)
    gs = gs_t.cpu().numpy()
    off = np.concatenate([[0], np.cumsum(gs)])
    m, k = x.shape
    n = A.shape[2]
    y, dx, dA = rd.ragged_dot_vjp(x, A, gs_t, dout)
    torch.cuda.synchronize()
    assert y.shape == (m, n) and dx.shape == (m, k) and dA.shape == A.shape

    rng = np.random.default_rng(5)
    for gi in _sample_groups(gs):
        lo, hi = int(off[gi]), int(off[gi + 1])
        rows = np.unique(np.concatenate([[lo, hi - 1], rng.integers(lo, hi, size=min(24, hi - lo))]))
        rt = torch.from_numpy(rows).cuda()
        # forward and dlhs rows: torch fp32 on the device, and the numpy oracle on the same rows
        y_t = (x[rt].float() @ A[gi].float())
        dx_t = (dout[rt].float() @ A[gi].float().T)
        util.assert_close_rows(util.to_np(y[rt]), util.to_np(y_t.to(torch.bfloat16)), len(rows), util.BF16_EPS, f"y g{gi}")
        util.assert_close_rows(util.to_np(dx[rt]), util.to_np(dx_t.to(torch.bfloat16)), len(rows), util.BF16_EPS, f"dlhs g{gi}")
        few = rows[:4]
        ft = torch.from_numpy(few).cuda()
        A_np = util.to_np(A[gi])
        y_o = oracle.gmm(util.to_np(x[ft]), A_np[None], [len(few)])
        dx_o = oracle.gmm(util.to_np(dout[ft]), A_np[None], [len(few)], trans_rhs=True)
        util.assert_close_rows(util.to_np(y[ft]), y_o, len(few), util.BF16_EPS, f"y vs oracle g{gi}")
        util.assert_close_rows(util.to_np(dx[ft]), dx_o, len(few), util.BF16_EPS, f"dlhs vs oracle g{gi}")
        # drhs of the whole group against torch fp32, and a corner block against the oracle
        dA_t = (x[lo:hi].float().T @ dout[lo:hi].float()).to(torch.bfloat16)
        util.assert_close_groups(util.to_np(dA[gi])[None], util.to_np(dA_t)[None], np.array([True]), util.TGMM_BF16_EPS, f"drhs g{gi}")
        blk = oracle.tgmm(util.to_np(x[lo:hi, :64]), util.to_np(dout[lo:hi, :48]), [hi - lo])
        util.assert_close_groups(util.to_np(dA[gi, :64, :48])[None], blk, np.array([True]), util.TGMM_BF16_EPS, f"drhs vs oracle g{gi}")

    empty = np.flatnonzero(gs == 0)
    if empty.size:
        assert not torch.any(dA[torch.from_numpy(empty).cuda()]).item(), "weights cotangent of empty groups must be zero"
    assert int(off[-1]) == m  # these two workloads fill every row

    # adjoint identity, accumulated in float64 on the device (bf16 outputs: agreement to ~1e-3 relative)
    s_y = torch.sum(dout.double() * y.double()).item()
    s_x = torch.sum(dx.double() * x.double()).item()
    s_A = sum(torch.sum(dA[i].double() * A[i].double()).item() for i in range(A.shape[0]))
    scale = torch.sum(dout.double().abs() * y.double().abs()).item()
    assert abs(s_y - s_x) <= 2e-3 * scale and abs(s_y - s_A) <= 2e-3 * scale, (s_y, s_x, s_A, scale)


def test_full_size_forward_with_tail_and_scaling():
    """Mixtral shape with the last group shortened: the tail must be exactly zero; doubling x doubles y exactly."""
    print("full size tail", flush=True)
    x, A, _, gs_t = workloads.make_inputs("mixtral_fwd")
    gs = gs_t.clone()
    gs[-1] -= 1000
    y = rd.ragged_dot(x, A, gs)
    total = int(gs.sum().item())
    assert not torch.any(y[total:]).item()
    assert torch.any(y[total - 1]).item()
    y2 = rd.ragged_dot(x * 2, A, gs)
    assert torch.equal(y2.float(), y.float() * 2)
