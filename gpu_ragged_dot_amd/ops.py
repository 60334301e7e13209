"""``ragged_dot`` / ``trans_ragged_dot`` with the reference's Python signature, running on HIP kernels.

Mirrors gpu_ragged_dot.py:345-454 (``gmm``, ``tgmm``, their aliases and the custom VJP).  Arrays are
``torch.Tensor`` on a ROCm device: torch supplies device memory and the stream, nothing else - every product is
computed by ``csrc/libragged_dot_hip.so`` through its C ABI.
"""

from __future__ import annotations

import ctypes
from typing import Optional

import torch

from . import _capi, planner
from .planner import CHUNK_M, DEFAULT_BLOCK_K, DEFAULT_BLOCK_M, DEFAULT_BLOCK_N

__all__ = ["gmm", "tgmm", "ragged_dot", "trans_ragged_dot", "ragged_dot_vjp", "make_group_metadata"]

_DTYPES = {torch.bfloat16: _capi.RD_DTYPE_BF16, torch.float32: _capi.RD_DTYPE_F32,
           torch.float8_e4m3fn: _capi.RD_DTYPE_F8E4M3_BF16, torch.float16: _capi.RD_DTYPE_F16}


def _out_dtype(t: torch.Tensor) -> torch.dtype:
    """The output has the operands' element type (gpu_ragged_dot.py:210,324); float8 operands, which the reference does
    not have, give bfloat16 (jax.lax.ragged_dot with preferred_element_type=bfloat16)."""
    return torch.bfloat16 if t.dtype == torch.float8_e4m3fn else t.dtype


def _dtype_code(t: torch.Tensor, compute_dtype, acc_dtype) -> int:
    """Element-type code for the C ABI from the storage dtype and the reference's ``compute_dtype``
    (gpu_ragged_dot.py:116-119, 145: operands are cast to compute_dtype before the dot; None = the storage dtype)."""
    if t.dtype not in _DTYPES:
        raise TypeError(f"unsupported dtype {t.dtype}; operands are bfloat16, float16, float32 or float8_e4m3fn")
    if acc_dtype not in (None, torch.float32):
        raise NotImplementedError("accumulation is always float32 on the matrix cores")
    if t.dtype == torch.float8_e4m3fn:
        if compute_dtype not in (None, torch.bfloat16, torch.float32, torch.float8_e4m3fn):
            raise NotImplementedError(f"no kernel for compute_dtype={compute_dtype} on float8 operands")
        return _capi.RD_DTYPE_F8E4M3_BF16  # float8 products are exact in every one of these types; accumulation is fp32
    if compute_dtype is None or compute_dtype == t.dtype:
        return _DTYPES[t.dtype]
    if t.dtype == torch.float32 and compute_dtype == torch.bfloat16:
        return _capi.RD_DTYPE_F32_BF16  # rounded to bf16 on the way to the bf16 matrix cores, float32 out
    if t.dtype == torch.float16 and compute_dtype == torch.float32:
        return _capi.RD_DTYPE_F16  # as for bfloat16 below: products of float16 values are exact in fp32
    if t.dtype == torch.bfloat16 and compute_dtype == torch.float32:
        # widening bf16 operands changes nothing: their products are exact in fp32 and accumulation is fp32 anyway
        return _capi.RD_DTYPE_BF16
    raise NotImplementedError(f"no kernel for compute_dtype={compute_dtype} on {t.dtype} operands")


def _aligned16(*tensors: torch.Tensor) -> bool:
    """The fast tile shapes move 16 bytes at a time: every buffer must start on a 16-byte boundary (a view at an odd
    element offset does not, however contiguous it is)."""
    return all(t.data_ptr() % 16 == 0 for t in tensors)


def _check_device(*tensors: torch.Tensor) -> torch.device:
    dev = tensors[0].device
    if dev.type != "cuda":
        raise RuntimeError(
            "ragged_dot runs on a ROCm device only (tensors must be on 'cuda'); there is no CPU path. "
            "interpret=True of the reference (the Pallas interpreter) has no counterpart here."
        )
    for t in tensors:
        if t.device != dev:
            raise RuntimeError("all operands must live on the same device")
    return dev


def _group_sizes_i32(group_sizes, dev: torch.device) -> torch.Tensor:
    gs = torch.as_tensor(group_sizes)
    if gs.dtype != torch.int32:
        gs = gs.to(torch.int32)
    return gs.to(dev).contiguous()


def _stream_ptr(dev: torch.device) -> int:
    return torch.cuda.current_stream(dev).cuda_stream


def _plan_ref(plan: Optional[_capi.Plan]):
    return ctypes.byref(plan) if plan is not None else None


def _group_offset(group_offset) -> int:
    """``group_offset`` as a host integer (None = 0; a one-element tensor is read back, which synchronises)."""
    if group_offset is None:
        return 0
    if isinstance(group_offset, torch.Tensor):
        assert group_offset.numel() == 1, "group_offset holds one group index"
        return int(group_offset.item())
    return int(group_offset)


def _gmm_fwd(x, A, group_sizes, block_m, block_k, block_n, trans_rhs, interpret, compute_dtype, acc_dtype, chunk_m,
             plan: Optional[_capi.Plan] = None, group_offset=None) -> torch.Tensor:
    """gpu_ragged_dot.py:171-228 (_gpu_gmm_fwd): checks, planning, one call across the C ABI.

    ``group_offset`` (jax.lax.ragged_dot's parameter; not in the reference): A holds the groups
    [group_offset, group_offset + A.shape[0]) of the ones group_sizes describes; rows of the others come out zero."""
    if interpret:
        raise NotImplementedError("interpret=True (Pallas interpreter) has no counterpart; kernels run on the GPU only")
    assert A.ndim == 3 and x.ndim == 2, f"but {A.ndim=} {x.ndim=}"  # :188
    gs_host_shape = tuple(torch.as_tensor(group_sizes).shape)
    g_first = _group_offset(group_offset)
    if group_offset is None:
        assert tuple(A.shape[:1]) == gs_host_shape, f"{A.shape[:1]=} != {gs_host_shape=}"  # :189
    else:
        assert len(gs_host_shape) == 1 and 0 <= g_first and g_first + A.shape[0] <= gs_host_shape[0], \
            f"groups [{g_first}, {g_first}+{A.shape[0]}) are not within {gs_host_shape=}"
    m, k = x.shape
    g_local, g = A.shape[0], gs_host_shape[0]
    n = A.shape[-1] if not trans_rhs else A.shape[-2]  # :190
    k_rhs = A.shape[-2] if not trans_rhs else A.shape[-1]
    assert k_rhs == k, f"contraction mismatch: x has k={k}, A has {k_rhs}"
    assert chunk_m >= 1
    planner.normalize_gmm_blocks(block_m, block_k, block_n, m, k, n)  # validates the request like :194-197
    dev = _check_device(x, A)
    code = _dtype_code(x, compute_dtype, acc_dtype)
    if A.dtype != x.dtype:
        raise TypeError(f"x is {x.dtype} but A is {A.dtype}")
    x, A = x.contiguous(), A.contiguous()
    gs = _group_sizes_i32(group_sizes, dev)
    y = torch.empty((m, n), dtype=_out_dtype(x), device=dev)  # :210
    if plan is None:
        plan = planner.select_plan(_capi.OP_GMM_TRANS if trans_rhs else _capi.OP_GMM, m, k, n, g, block_m, block_k, block_n,
                                   dtype=code, aligned=_aligned16(x, A, y))
    if (g_first, g_local) != (0, g) and plan.decode_nb:
        plan = _capi.Plan(plan.variant, plan.group_m, 0, plan.group_n, plan.split_k)  # streaming kernels: all groups only
    ws_bytes = _capi.lib.rd_gmm_workspace_bytes(m, g, _plan_ref(plan))
    ws = torch.empty(max(ws_bytes, 256), dtype=torch.uint8, device=dev)
    with torch.cuda.device(dev):
        _capi.check(
            _capi.lib.rd_gmm_sharded(_stream_ptr(dev), x.data_ptr(), A.data_ptr(), gs.data_ptr(), y.data_ptr(), m, k, n,
                                     g, g_first, g_local, int(bool(trans_rhs)), code, _plan_ref(plan), ws.data_ptr(),
                                     ws.numel())
        )
    return y


def _tgmm_fwd(x, y, group_sizes, block_m, block_k, block_n, interpret, compute_dtype, acc_dtype, chunk_m,
              plan: Optional[_capi.Plan] = None, group_offset=None, num_actual_groups=None) -> torch.Tensor:
    """gpu_ragged_dot.py:287-342 (_gpu_tgmm_fwd).  With ``group_offset`` / ``num_actual_groups`` only the slices of the
    groups [group_offset, group_offset + num_actual_groups) are computed: out[i] belongs to group group_offset + i."""
    del chunk_m  # :303
    if interpret:
        raise NotImplementedError("interpret=True (Pallas interpreter) has no counterpart; kernels run on the GPU only")
    assert y.ndim == 2 and x.ndim == 2 and x.shape[0] == y.shape[0]  # :304
    (m, k), n = x.shape, y.shape[-1]
    gs_t = torch.as_tensor(group_sizes)
    g = gs_t.numel()
    planner.normalize_tgmm_blocks(block_m, block_k, block_n, m, k, n)  # :308-314
    dev = _check_device(x, y)
    code = _dtype_code(x, compute_dtype, acc_dtype)
    if y.dtype != x.dtype:
        raise TypeError(f"x is {x.dtype} but y is {y.dtype}")
    x, y = x.contiguous(), y.contiguous()
    gs = _group_sizes_i32(gs_t, dev)
    g_first = _group_offset(group_offset)
    g_local = g - g_first if num_actual_groups is None else int(num_actual_groups)
    assert 0 <= g_first and g_local >= 1 and g_first + g_local <= g, f"groups [{g_first}, {g_first}+{g_local}) are not within {g}"
    out = torch.empty((g_local, k, n), dtype=_out_dtype(x), device=dev)  # :324
    if plan is None:
        plan = planner.select_plan(_capi.OP_TGMM, m, k, n, g, block_m, block_k, block_n, dtype=code,
                                   aligned=_aligned16(x, y, out))
    ws_bytes = _capi.lib.rd_tgmm_workspace_bytes(m, g, _plan_ref(plan))
    ws = torch.empty(max(ws_bytes, 256), dtype=torch.uint8, device=dev)
    with torch.cuda.device(dev):
        _capi.check(
            _capi.lib.rd_tgmm_sharded(_stream_ptr(dev), x.data_ptr(), y.data_ptr(), gs.data_ptr(), out.data_ptr(), m, k, n,
                                      g, g_first, g_local, code, _plan_ref(plan), ws.data_ptr(), ws.numel())
        )
    return out


class _GmmFn(torch.autograd.Function):
    """The custom VJP of gpu_ragged_dot.py:360-405, as a torch autograd node."""

    @staticmethod
    def forward(ctx, x, A, group_sizes, hp):
        ctx.hp = hp
        ctx.save_for_backward(x, A, group_sizes)  # residuals (x, A, group_sizes), :227
        return _gmm_fwd(x, A, group_sizes, **hp)

    @staticmethod
    def backward(ctx, do):
        x, A, group_sizes = ctx.saved_tensors
        hp = dict(ctx.hp)
        trans_rhs = hp.pop("trans_rhs")
        hp.pop("plan", None)
        do = do.contiguous()
        dx = dA = None
        if ctx.needs_input_grad[0]:
            dx = _gmm_fwd(do, A, group_sizes, **hp, trans_rhs=not trans_rhs)  # :400 (rows of groups outside A's slice: zero)
        if ctx.needs_input_grad[1]:
            thp = {k_: v for k_, v in hp.items()}
            thp["num_actual_groups"] = A.shape[0]
            dA = _tgmm_fwd(x, do, group_sizes, **thp) if not trans_rhs else _tgmm_fwd(do, x, group_sizes, **thp)  # :401
        return dx, dA, None, None  # group_sizes gets no cotangent, :402


class _TgmmFn(torch.autograd.Function):
    """tgmm with the VJP gpu_ragged_dot.py:431-450 intends: dx = gmm(y, do, trans_rhs=True), dy = gmm(x, do)."""

    @staticmethod
    def forward(ctx, x, y, group_sizes, hp):
        ctx.hp = hp
        ctx.save_for_backward(x, y, group_sizes)
        return _tgmm_fwd(x, y, group_sizes, **hp)

    @staticmethod
    def backward(ctx, do):
        x, y, group_sizes = ctx.saved_tensors
        hp = dict(ctx.hp)
        hp.pop("plan", None)
        hp.pop("num_actual_groups", None)  # do has that many slices; group_offset says which groups they are
        do = do.contiguous()
        dx = dy = None
        if ctx.needs_input_grad[0]:
            dx = _gmm_fwd(y, do, group_sizes, **hp, trans_rhs=True)
        if ctx.needs_input_grad[1]:
            dy = _gmm_fwd(x, do, group_sizes, **hp, trans_rhs=False)
        return dx, dy, None, None


def gmm(
    x: torch.Tensor,  # [m, k]
    A: torch.Tensor,  # [g, k, n]  ([g, n, k] with trans_rhs)
    group_sizes,  # [g]
    block_m: int = DEFAULT_BLOCK_M,
    block_k: int = DEFAULT_BLOCK_K,
    block_n: int = DEFAULT_BLOCK_N,
    trans_rhs: bool = False,
    interpret: bool = False,
    compute_dtype=None,
    acc_dtype=torch.float32,
    num_warps: Optional[int] = None,
    num_stages: Optional[int] = None,
    chunk_m: int = CHUNK_M,
    group_offset=None,
) -> torch.Tensor:
    """Ragged dot corresponding to jax.lax.ragged_dot: (m, k) x (g, k, n) -> (m, n).  gpu_ragged_dot.py:362-380.

    ``num_warps`` / ``num_stages`` are Triton knobs of the reference and are accepted and ignored; ``chunk_m`` is
    validated only (the kernels split groups by their own tile height).  ``group_offset`` (after the reference's
    parameters; jax.lax.ragged_dot's own keyword): A holds only the groups [group_offset, group_offset + A.shape[0])
    of those in group_sizes - an expert-parallel rank's slice; rows of the other groups are zero.
    """
    del num_warps, num_stages
    hp = dict(block_m=block_m, block_k=block_k, block_n=block_n, trans_rhs=trans_rhs, interpret=interpret,
              compute_dtype=compute_dtype, acc_dtype=acc_dtype, chunk_m=chunk_m)
    if group_offset is not None:
        hp["group_offset"] = _group_offset(group_offset)
    if torch.is_grad_enabled() and (x.requires_grad or A.requires_grad):
        if x.dtype == torch.float8_e4m3fn:
            raise NotImplementedError("float8 operands are forward only: their cotangents are bfloat16, differentiate a bfloat16 copy")
        gs = _group_sizes_i32(group_sizes, x.device)
        return _GmmFn.apply(x, A, gs, hp)
    return _gmm_fwd(x, A, group_sizes, **hp)


def tgmm(
    x: torch.Tensor,  # [m, k]
    y: torch.Tensor,  # [m, n]
    group_sizes,  # [g]
    block_m: int = DEFAULT_BLOCK_M,
    block_k: int = DEFAULT_BLOCK_K,
    block_n: int = DEFAULT_BLOCK_N,
    interpret: bool = False,
    compute_dtype=None,
    acc_dtype=torch.float32,
    num_warps: Optional[int] = None,
    num_stages: Optional[int] = None,
    chunk_m: int = CHUNK_M,
    group_offset=None,
    num_actual_groups: Optional[int] = None,
) -> torch.Tensor:
    """Transposed ragged dot: (m, k) x (m, n) -> (g, k, n).  gpu_ragged_dot.py:411-428.  With ``group_offset`` /
    ``num_actual_groups`` only the slices of the groups [group_offset, group_offset + num_actual_groups) are computed."""
    del num_warps, num_stages
    hp = dict(block_m=block_m, block_k=block_k, block_n=block_n, interpret=interpret, compute_dtype=compute_dtype,
              acc_dtype=acc_dtype, chunk_m=chunk_m)
    if group_offset is not None or num_actual_groups is not None:
        hp["group_offset"] = _group_offset(group_offset)
        hp["num_actual_groups"] = num_actual_groups
    if torch.is_grad_enabled() and (x.requires_grad or y.requires_grad):
        gs = _group_sizes_i32(group_sizes, x.device)
        return _TgmmFn.apply(x, y, gs, hp)
    return _tgmm_fwd(x, y, group_sizes, **hp)


ragged_dot = gmm  # gpu_ragged_dot.py:406
trans_ragged_dot = tgmm  # gpu_ragged_dot.py:454


def ragged_dot_vjp(x, A, group_sizes, dout, trans_rhs: bool = False, **hp):
    """Forward plus the VJP rule of gpu_ragged_dot.py:383-402 in one call: returns (y, dx, dA)."""
    kw = dict(block_m=DEFAULT_BLOCK_M, block_k=DEFAULT_BLOCK_K, block_n=DEFAULT_BLOCK_N, interpret=False,
              compute_dtype=None, acc_dtype=torch.float32, chunk_m=CHUNK_M)
    kw.update(hp)
    y = _gmm_fwd(x, A, group_sizes, **kw, trans_rhs=trans_rhs)
    dx = _gmm_fwd(dout, A, group_sizes, **kw, trans_rhs=not trans_rhs)
    dA = _tgmm_fwd(x, dout, group_sizes, **kw) if not trans_rhs else _tgmm_fwd(dout, x, group_sizes, **kw)
    return y, dx, dA


def make_group_metadata(group_sizes, m: int, chunk_m: int = CHUNK_M):
    """The scheduling map of gpu_ragged_dot.py:70-90, computed on the device.

    Returns (group_offsets[g], row_it2group[U], row_it2it_in_group[U], total_row_its[1]) as int32 device tensors.
    """
    gs_t = torch.as_tensor(group_sizes)
    if gs_t.device.type != "cuda":
        gs_t = gs_t.to("cuda")
    dev = gs_t.device
    gs = _group_sizes_i32(gs_t, dev)
    g = gs.numel()
    U = _capi.lib.rd_sched_map_len(m, g, chunk_m)
    if U < 0:
        _capi.check(U)
    offs = torch.empty(g, dtype=torch.int32, device=dev)
    t2g = torch.empty(U, dtype=torch.int32, device=dev)
    t2it = torch.empty(U, dtype=torch.int32, device=dev)
    total = torch.empty(1, dtype=torch.int32, device=dev)
    with torch.cuda.device(dev):
        _capi.check(
            _capi.lib.rd_sched_map(_stream_ptr(dev), gs.data_ptr(), g, m, chunk_m, offs.data_ptr(), t2g.data_ptr(),
                                   t2it.data_ptr(), total.data_ptr())
        )
    return offs, t2g, t2it, total
