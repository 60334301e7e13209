"""Host-side planning for ragged_dot: the reference's block-size rules and the choice of a compiled tile shape.

The reference turns ``block_m/k/n`` into Triton block shapes (gpu_ragged_dot.py:194-197, 308-314).  Here the
kernels come in a fixed set of compiled tile shapes, so the same keywords act as a request: the defaults mean
"use the tuned table or the library's shape heuristic", anything else picks the nearest compiled shape.
"""

from __future__ import annotations

import json
import math
import os
from typing import Optional

from . import _capi

DEFAULT_BLOCK_M = 64  # gpu_ragged_dot.py:34-36
DEFAULT_BLOCK_N = 64
DEFAULT_BLOCK_K = 64
CHUNK_M = 512  # gpu_ragged_dot.py:42

TUNED_PLANS_PATH = os.environ.get(
    "RAGGED_DOT_TUNED_PLANS", os.path.join(os.path.dirname(os.path.abspath(__file__)), "tuned_plans.json")
)


def cdiv(a: int, b: int) -> int:
    return -(-a // b)


def next_power_of_2(x: int) -> int:
    if x < 0:
        raise ValueError("next_power_of_2 needs a non-negative integer")
    return 1 if x == 0 else 1 << (int(x) - 1).bit_length()


def normalize_gmm_blocks(block_m: int, block_k: int, block_n: int, m: int, k: int, n: int) -> tuple[int, int, int]:
    """gpu_ragged_dot.py:194-197."""
    bm, bk, bn = (next_power_of_2(min(b, s)) for b, s in zip((block_m, block_k, block_n), (m, k, n)))
    return bm, max(bk, 16), max(bn, 16)


def normalize_tgmm_blocks(block_m: int, block_k: int, block_n: int, m: int, k: int, n: int) -> tuple[int, int, int]:
    """gpu_ragged_dot.py:308-314."""
    block_m, block_n = min(block_m, m), min(block_n, n)
    bm, bk, bn = (max(next_power_of_2(min(b, s)), 16) for b, s in zip((block_m, block_k, block_n), (m, k, n)))
    return bm, bk, bn


_VARIANTS: Optional[list] = None
_TUNED: Optional[dict] = None


def compiled_variants() -> list:
    global _VARIANTS
    if _VARIANTS is None:
        _VARIANTS = _capi.variants()
    return _VARIANTS


def variant_id(name: str) -> int:
    for v in compiled_variants():
        if v.name.decode() == name:
            return v.id
    raise KeyError(f"no compiled tile variant named {name!r}")


def tuned_plans() -> dict:
    global _TUNED
    if _TUNED is None:
        try:
            with open(TUNED_PLANS_PATH) as f:
                _TUNED = json.load(f)
        except FileNotFoundError:
            _TUNED = {}
    return _TUNED


def plan_key(op: int, m: int, k: int, n: int, g: int) -> str:
    return f"{('gmm', 'gmm_t', 'tgmm')[op]}:m{m}:k{k}:n{n}:g{g}"


def select_plan(
    op: int,
    m: int,
    k: int,
    n: int,
    g: int,
    block_m: int = DEFAULT_BLOCK_M,
    block_k: int = DEFAULT_BLOCK_K,
    block_n: int = DEFAULT_BLOCK_N,
    dtype: int = _capi.RD_DTYPE_BF16,
    aligned: bool = True,
) -> _capi.Plan:
    """Plan for op (0 gmm, 1 gmm with trans_rhs, 2 tgmm) on a problem of this shape and element type.

    ``aligned``: every buffer of the call starts on a 16-byte boundary.  When one does not, the plan is the
    element-granular tile shape of that element type, whatever the shape, the tuned table or block_* ask for."""
    if not aligned and dtype != _capi.RD_DTYPE_F32:
        for v in compiled_variants():
            if v.dtype == dtype and not v.vec:
                return _capi.Plan(v.id)
        raise _capi.RaggedDotError(_capi.RD_ERR_UNSUPPORTED, "no any-alignment tile shape compiled in for this dtype")
    if dtype != _capi.RD_DTYPE_BF16:
        return _capi.default_plan(op, m, k, n, g, dtype)  # the library's own choice: nothing to tune
    vec = k % 8 == 0 and n % 8 == 0
    explicit = (block_m, block_k, block_n) != (DEFAULT_BLOCK_M, DEFAULT_BLOCK_K, DEFAULT_BLOCK_N)
    entry = tuned_plans().get(plan_key(op, m, k, n, g))
    if entry is not None and vec and not explicit:
        return _capi.Plan(variant_id(entry["variant"]), int(entry.get("group_m", 0)), int(entry.get("decode_nb", 0)),
                          int(entry.get("group_n", 0)))
    plan = _capi.default_plan(op, m, k, n, g)
    if explicit and not plan.decode_nb:
        # explicit request: nearest compiled shape.  For tgmm the output tile is (block_k, block_n).
        want_rows = block_k if op == _capi.OP_TGMM else block_m
        best, best_d = None, None
        for v in compiled_variants():
            if bool(v.vec) != vec or v.dtype != _capi.RD_DTYPE_BF16:
                continue
            d = abs(math.log2(v.tile_m / max(want_rows, 1))) + abs(math.log2(v.tile_n / max(block_n, 1)))
            if best_d is None or d < best_d:
                best, best_d = v.id, d
        if best is not None:
            plan.variant = best
    return plan
