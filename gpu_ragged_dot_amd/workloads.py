"""Seeded synthetic inputs for the benchmark / parity configurations (numpy PCG64 for the group sizes, so they are
bit-identical on every machine; tensors are drawn on the device from a seeded torch generator)."""

from __future__ import annotations

from dataclasses import dataclass

import numpy as np
import torch


@dataclass(frozen=True)
class Workload:
    name: str
    m: int
    k: int
    n: int
    g: int
    backward: bool  # forward + VJP, or forward only
    description: str


WORKLOADS = {
    "tiny": Workload("tiny", 512, 256, 512, 4, True, "tiny fwd+VJP, multinomial group sizes"),
    "mixtral_fwd": Workload("mixtral_fwd", 16384, 4096, 14336, 8, False, "Mixtral-8x7B up-projection, 8192 tokens x top-2, forward"),
    "mixtral_fwd_bwd": Workload("mixtral_fwd_bwd", 16384, 4096, 14336, 8, True, "Mixtral-8x7B up-projection, forward + dlhs + drhs"),
    "deepseek_fwd_bwd": Workload("deepseek_fwd_bwd", 32768, 7168, 2048, 256, True, "DeepSeek-V3 routed experts, Zipf-skewed sizes, ~10% empty, forward + backward"),
    "decode": Workload("decode", 64, 2048, 768, 128, False, "Qwen3-30B-A3B decode, 8 tokens x top-8, forward only"),
    # the other projections of the same layers and a prefill batch (not benchmark configurations: shapes for the tuner,
    # `python -m gpu_ragged_dot_amd.tune --workload <name> --write`, and for `bench.py --workload <name> --only`)
    "mixtral_down_fwd_bwd": Workload("mixtral_down_fwd_bwd", 16384, 14336, 4096, 8, True, "Mixtral-8x7B down-projection, same routing, forward + backward"),
    "deepseek_down_fwd_bwd": Workload("deepseek_down_fwd_bwd", 32768, 2048, 7168, 256, True, "DeepSeek-V3 routed experts' down-projection, same routing, forward + backward"),
    "qwen3_prefill_fwd_bwd": Workload("qwen3_prefill_fwd_bwd", 32768, 2048, 768, 128, True, "Qwen3-30B-A3B expert up-projection, 4096 tokens x top-8, forward + backward"),
    "qwen3_prefill_down_fwd_bwd": Workload("qwen3_prefill_down_fwd_bwd", 32768, 768, 2048, 128, True, "Qwen3-30B-A3B expert down-projection, 4096 tokens x top-8, forward + backward"),
}


def top_k_counts(seed: int, tokens: int, g: int, top: int) -> np.ndarray:
    """Tokens per expert when every token goes to its `top` largest of g seeded Gaussian router logits."""
    rng = np.random.default_rng(seed)
    logits = rng.standard_normal((tokens, g), dtype=np.float32)
    idx = np.argpartition(-logits, top - 1, axis=1)[:, :top]
    return np.bincount(idx.ravel(), minlength=g).astype(np.int32)


def zipf_counts(seed: int, total: int, g: int, s: float, n_empty: int) -> np.ndarray:
    """Multinomial over a randomly permuted Zipf(s) law with n_empty groups forced to probability zero."""
    rng = np.random.default_rng(seed)
    ranks = rng.permutation(g) + 1
    p = ranks.astype(np.float64) ** -s
    p[rng.choice(g, size=n_empty, replace=False)] = 0.0
    p /= p.sum()
    return rng.multinomial(total, p).astype(np.int32)


def group_sizes(name: str) -> np.ndarray:
    if name == "tiny":
        return np.random.default_rng(0).multinomial(512, [0.25] * 4).astype(np.int32)
    if name in ("mixtral_fwd", "mixtral_fwd_bwd", "mixtral_down_fwd_bwd"):
        return top_k_counts(1, 8192, 8, 2)
    if name in ("deepseek_fwd_bwd", "deepseek_down_fwd_bwd"):
        return zipf_counts(2, 32768, 256, 1.1, 26)
    if name in ("qwen3_prefill_fwd_bwd", "qwen3_prefill_down_fwd_bwd"):
        return top_k_counts(4, 4096, 128, 8)
    if name == "decode":
        return top_k_counts(3, 8, 128, 8)
    raise KeyError(name)


def make_inputs(name: str, device="cuda", dtype=torch.bfloat16, seed: int = 100):
    """(x[m,k] ~ N(0,1), A[g,k,n] ~ N(0, 1/k), dout[m,n] ~ N(0,1) or None, group_sizes int32[g]) on `device`."""
    w = WORKLOADS[name]
    gen = torch.Generator(device=device)
    gen.manual_seed(seed)
    x = torch.randn((w.m, w.k), generator=gen, device=device, dtype=torch.float32).to(dtype)
    A = torch.empty((w.g, w.k, w.n), device=device, dtype=dtype)
    scale = 1.0 / float(np.sqrt(w.k))
    for gi in range(w.g):  # group by group: keeps the fp32 staging buffer small for the 7.5 GB weight tensor
        A[gi] = (torch.randn((w.k, w.n), generator=gen, device=device, dtype=torch.float32) * scale).to(dtype)
    dout = None
    if w.backward:
        dout = torch.randn((w.m, w.n), generator=gen, device=device, dtype=torch.float32).to(dtype)
    gs = torch.from_numpy(group_sizes(name)).to(device)
    return x, A, dout, gs


def flops(name: str) -> float:
    """Algorithmic FLOPs of one step: 2 * sum(group_sizes) * k * n per product; forward = 1, forward+backward = 3."""
    w = WORKLOADS[name]
    rows = int(group_sizes(name).sum())
    return 2.0 * rows * w.k * w.n * (3 if w.backward else 1)


def algorithmic_bytes(name: str, elem: int = 2) -> dict:
    """Bytes each product must move: every operand read once, output written once; weights of empty groups are
    not read by gmm; tgmm writes all g*k*n."""
    w = WORKLOADS[name]
    gs = group_sizes(name)
    nonempty = int((gs > 0).sum())
    xb, yb = w.m * w.k * elem, w.m * w.n * elem
    wb_read, wb_all = nonempty * w.k * w.n * elem, w.g * w.k * w.n * elem
    out = {"fwd": xb + wb_read + yb}
    if w.backward:
        out["dlhs"] = yb + wb_read + xb
        out["drhs"] = xb + yb + wb_all
    out["weights_read"] = wb_read
    return out
