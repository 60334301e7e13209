"""``ragged_dot`` / ``trans_ragged_dot`` for JAX arrays: the reference's own surface over the HIP kernels.

This is the literal drop-in for ``gpu_ragged_dot.py``: the same names (``gmm``, ``tgmm``, ``ragged_dot``,
``trans_ragged_dot``), the same positional order and defaults, ``jax.custom_vjp`` with every hyper-parameter
non-differentiable over ``jax.jit`` with the hyper-parameters static (gpu_ragged_dot.py:347-361, 383-405, 409-428) -
only the kernel call differs: ``jax.ffi.ffi_call`` into the XLA FFI handlers of ``csrc/rd_xla_ffi.cc`` where the
reference has ``pl.pallas_call`` (:217-226, :331-340).

Importing this module needs ``jax`` (with a ROCm PJRT plugin) and ``librd_xla_ffi.so`` built by
``make -C gpu_ragged_dot_amd/csrc xla_ffi XLA_FFI_INCLUDE=$(python -c 'import jax.ffi; print(jax.ffi.include_dir())')``.
Neither exists in an image without JAX; there it raises ImportError and nothing else in the package depends on it.
It has not been run: the torch front end (``ops.py``) is the one the parity tests exercise through the same C ABI.

Differences from the reference, all deliberate:
* ``interpret=True`` raises (no CPU path); ``num_warps`` / ``num_stages`` are accepted and ignored;
* ``block_m/k/n`` choose among the compiled tile shapes (``planner.select_plan``) instead of sizing a Triton block;
* the VJP of ``tgmm`` uses ``dy = gmm(x, do)``: gpu_ragged_dot.py:447-449 writes ``tgmm(x, do)``, which cannot trace
  (a 3-D ``do`` fails the assert of :304), and its bwd declares a leading ``group_sizes`` parameter (:432) that
  ``custom_vjp`` never passes.
"""

from __future__ import annotations

import ctypes
import os
from functools import partial
from typing import Optional

import jax  # ImportError here is the gate: no JAX, no adapter
import jax.numpy as jnp
import numpy as np

from . import _capi, planner
from .planner import CHUNK_M, DEFAULT_BLOCK_K, DEFAULT_BLOCK_M, DEFAULT_BLOCK_N

__all__ = ["gmm", "tgmm", "ragged_dot", "trans_ragged_dot"]

_SHIM_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc", "librd_xla_ffi.so")
if not os.path.exists(_SHIM_PATH):
    raise ImportError(f"{_SHIM_PATH} is missing: build it with `make -C {os.path.dirname(_SHIM_PATH)} xla_ffi "
                      "XLA_FFI_INCLUDE=<jax.ffi.include_dir()>`")
_shim = ctypes.CDLL(_SHIM_PATH)
for _target, _symbol in (("rd_gmm", "RdGmm"), ("rd_tgmm", "RdTgmm")):
    jax.ffi.register_ffi_target(_target, jax.ffi.pycapsule(getattr(_shim, _symbol)), platform="ROCM")


def _dtype_code(dtype, compute_dtype, acc_dtype) -> int:
    """RD_DTYPE_* from the storage dtype and compute_dtype (gpu_ragged_dot.py:116-119); same rules as ops._dtype_code."""
    if acc_dtype not in (None, jnp.float32, np.float32):
        raise NotImplementedError("accumulation is always float32 on the matrix cores")
    dtype = jnp.dtype(dtype)
    compute = dtype if compute_dtype is None else jnp.dtype(compute_dtype)
    if dtype == jnp.bfloat16 and compute in (jnp.dtype(jnp.bfloat16), jnp.dtype(jnp.float32)):
        return _capi.RD_DTYPE_BF16  # widening bf16 operands changes nothing: exact products, fp32 accumulation
    if dtype == jnp.float16 and compute in (jnp.dtype(jnp.float16), jnp.dtype(jnp.float32)):
        return _capi.RD_DTYPE_F16  # as for bfloat16: products of float16 values are exact in fp32
    if dtype == jnp.float32 and compute == jnp.dtype(jnp.float32):
        return _capi.RD_DTYPE_F32
    if dtype == jnp.float32 and compute == jnp.dtype(jnp.bfloat16):
        return _capi.RD_DTYPE_F32_BF16
    if dtype == jnp.float8_e4m3fn and compute in (dtype, jnp.dtype(jnp.bfloat16), jnp.dtype(jnp.float32)):
        return _capi.RD_DTYPE_F8E4M3_BF16  # jax.lax.ragged_dot with preferred_element_type=bfloat16; forward only
    raise NotImplementedError(f"no kernel for compute_dtype={compute_dtype} on {dtype} operands")


def _out_dtype(dtype):
    """The result has the operands' element type (gpu_ragged_dot.py:210,324); float8 operands give bfloat16."""
    return jnp.bfloat16 if jnp.dtype(dtype) == jnp.float8_e4m3fn else dtype


def _plan_attrs(plan: _capi.Plan) -> dict:
    return dict(variant=np.int32(plan.variant), group_m=np.int32(plan.group_m), group_n=np.int32(plan.group_n),
                decode_nb=np.int32(plan.decode_nb), split_k=np.int32(plan.split_k))


def _workspace(nbytes: int) -> jax.ShapeDtypeStruct:
    # a second result that XLA allocates and the caller drops: the handlers never allocate
    return jax.ShapeDtypeStruct((max(int(nbytes), 256),), jnp.uint8)


def _gmm_fwd(x, A, group_sizes, block_m, block_k, block_n, trans_rhs, interpret, compute_dtype, acc_dtype, num_warps,
             num_stages, chunk_m):
    """Forward rule and primal body of gmm: gpu_ragged_dot.py:171-228 with the pallas_call replaced."""
    del num_warps, num_stages
    if interpret:
        raise NotImplementedError("interpret=True (Pallas interpreter) has no counterpart; kernels run on the GPU only")
    assert A.ndim == 3 and x.ndim == 2, f"but {A.ndim=} {x.ndim=}"  # :188
    assert A.shape[:1] == group_sizes.shape, f"{A.shape[:1]=} != {group_sizes.shape=}"  # :189
    (m, k), g = x.shape, A.shape[0]
    n = A.shape[-1] if not trans_rhs else A.shape[-2]  # :190
    assert (A.shape[-2] if not trans_rhs else A.shape[-1]) == k and A.dtype == x.dtype and chunk_m >= 1
    planner.normalize_gmm_blocks(block_m, block_k, block_n, m, k, n)  # validates like :194-197
    code = _dtype_code(x.dtype, compute_dtype, acc_dtype)
    plan = planner.select_plan(_capi.OP_GMM_TRANS if trans_rhs else _capi.OP_GMM, m, k, n, g, block_m, block_k, block_n,
                               dtype=code)  # XLA buffers are at least 16-byte aligned
    ws_bytes = _capi.lib.rd_gmm_workspace_bytes(m, g, ctypes.byref(plan))
    with jax.named_scope("gpu_gmm"):  # :216
        y, _ = jax.ffi.ffi_call("rd_gmm", (jax.ShapeDtypeStruct((m, n), _out_dtype(x.dtype)), _workspace(ws_bytes)))(
            x, A, group_sizes.astype(jnp.int32), trans_rhs=bool(trans_rhs), compute_bf16=code == _capi.RD_DTYPE_F32_BF16,
            chunk_m=np.int32(chunk_m), **_plan_attrs(plan))
    return y, (x, A, group_sizes)  # residuals, :227


def _tgmm_fwd(x, y, group_sizes, block_m, block_k, block_n, interpret, compute_dtype, acc_dtype, num_warps, num_stages,
              chunk_m):
    """Forward rule and primal body of tgmm: gpu_ragged_dot.py:287-342 with the pallas_call replaced."""
    del num_warps, num_stages
    if interpret:
        raise NotImplementedError("interpret=True (Pallas interpreter) has no counterpart; kernels run on the GPU only")
    assert y.ndim == 2 and x.ndim == 2 and x.shape[0] == y.shape[0]  # :304
    (m, k), n, g = x.shape, y.shape[-1], group_sizes.shape[0]
    assert y.dtype == x.dtype
    planner.normalize_tgmm_blocks(block_m, block_k, block_n, m, k, n)  # :308-314
    code = _dtype_code(x.dtype, compute_dtype, acc_dtype)
    plan = planner.select_plan(_capi.OP_TGMM, m, k, n, g, block_m, block_k, block_n, dtype=code)
    ws_bytes = _capi.lib.rd_tgmm_workspace_bytes(m, g, ctypes.byref(plan))
    with jax.named_scope("gpu_tgmm"):  # :330
        out, _ = jax.ffi.ffi_call("rd_tgmm", (jax.ShapeDtypeStruct((g, k, n), _out_dtype(x.dtype)), _workspace(ws_bytes)))(
            x, y, group_sizes.astype(jnp.int32), compute_bf16=code == _capi.RD_DTYPE_F32_BF16, chunk_m=np.int32(chunk_m),
            **_plan_attrs(plan))
    return out, (x, y, group_sizes)


NONDIFF_ARGNAMES = ("block_m", "block_k", "block_n", "interpret", "compute_dtype", "acc_dtype", "num_warps",
                    "num_stages", "chunk_m")  # gpu_ragged_dot.py:347-357


@partial(jax.custom_vjp, nondiff_argnames=NONDIFF_ARGNAMES + ("trans_rhs",))
@partial(jax.jit, static_argnums=list(range(3, 13)))
def gmm(
    x: jax.Array,  # [m, k]
    A: jax.Array,  # [g, k, n]  ([g, n, k] with trans_rhs)
    group_sizes: jax.Array,  # [g]
    block_m: int = DEFAULT_BLOCK_M,
    block_k: int = DEFAULT_BLOCK_K,
    block_n: int = DEFAULT_BLOCK_N,
    trans_rhs: bool = False,
    interpret: bool = False,
    compute_dtype: Optional["jnp.dtype"] = None,
    acc_dtype: Optional["jnp.dtype"] = jnp.float32,
    num_warps: int | None = None,
    num_stages: int | None = None,
    chunk_m: int = CHUNK_M,
) -> jax.Array:
    """Ragged dot corresponding to jax.lax.ragged_dot: (m, k) x (g, k, n) -> (m, n).  gpu_ragged_dot.py:362-380."""
    return _gmm_fwd(x, A, group_sizes, block_m, block_k, block_n, trans_rhs, interpret, compute_dtype, acc_dtype,
                    num_warps, num_stages, chunk_m)[0]


def _gmm_fwd_rule(x, A, group_sizes, block_m, block_k, block_n, trans_rhs, interpret, compute_dtype, acc_dtype,
                  num_warps, num_stages, chunk_m):
    return _gmm_fwd(x, A, group_sizes, block_m, block_k, block_n, trans_rhs, interpret, compute_dtype, acc_dtype,
                    num_warps, num_stages, chunk_m)


def _gmm_bwd_rule(block_m, block_k, block_n, trans_rhs, interpret, compute_dtype, acc_dtype, num_warps, num_stages,
                  chunk_m, res, do):
    """gpu_ragged_dot.py:383-402: non-differentiable arguments first, in the primal's positional order."""
    hp = dict(block_m=block_m, block_k=block_k, block_n=block_n, interpret=interpret, compute_dtype=compute_dtype,
              acc_dtype=acc_dtype, num_warps=num_warps, num_stages=num_stages, chunk_m=chunk_m)
    x, A, group_sizes = res
    dx = gmm(do, A, group_sizes, trans_rhs=not trans_rhs, **hp)  # :400
    dA = tgmm(do, x, group_sizes, **hp) if trans_rhs else tgmm(x, do, group_sizes, **hp)  # :401
    return dx, dA, None  # no cotangent for group_sizes, :402


gmm.defvjp(_gmm_fwd_rule, _gmm_bwd_rule)  # :405
ragged_dot = gmm  # :406


@partial(jax.custom_vjp, nondiff_argnames=NONDIFF_ARGNAMES)
@partial(jax.jit, static_argnums=list(range(3, 12)))
def tgmm(
    x: jax.Array,  # [m, k]
    y: jax.Array,  # [m, n]
    group_sizes: jax.Array,  # [g]
    block_m: int = DEFAULT_BLOCK_M,
    block_k: int = DEFAULT_BLOCK_K,
    block_n: int = DEFAULT_BLOCK_N,
    interpret: bool = False,
    compute_dtype: Optional["jnp.dtype"] = None,
    acc_dtype: Optional["jnp.dtype"] = jnp.float32,
    num_warps: int | None = None,
    num_stages: int | None = None,
    chunk_m: int = CHUNK_M,
) -> jax.Array:
    """Transposed ragged dot: (m, k) x (m, n) -> (g, k, n).  gpu_ragged_dot.py:411-428."""
    return _tgmm_fwd(x, y, group_sizes, block_m, block_k, block_n, interpret, compute_dtype, acc_dtype, num_warps,
                     num_stages, chunk_m)[0]


def _tgmm_bwd_rule(block_m, block_k, block_n, interpret, compute_dtype, acc_dtype, num_warps, num_stages, chunk_m, res,
                   do):
    """What gpu_ragged_dot.py:431-450 intends, with the arity and the second product put right."""
    hp = dict(block_m=block_m, block_k=block_k, block_n=block_n, interpret=interpret, compute_dtype=compute_dtype,
              acc_dtype=acc_dtype, num_warps=num_warps, num_stages=num_stages, chunk_m=chunk_m)
    x, y, group_sizes = res
    dx = gmm(y, do, group_sizes, trans_rhs=True, **hp)   # rows of group g: y_g . do[g]^T
    dy = gmm(x, do, group_sizes, trans_rhs=False, **hp)  # rows of group g: x_g . do[g]
    return dx, dy, None


tgmm.defvjp(_tgmm_fwd, _tgmm_bwd_rule)
trans_ragged_dot = tgmm  # :454
