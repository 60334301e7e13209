"""Token routing around ``ragged_dot`` for a mixture of experts, on the device.

``ragged_dot`` takes rows sorted by group; the reference leaves producing them to its caller (its tests build sorted
rows directly, tests.py:51-71).  This module is that caller's side, each function one call across the C ABI
(``rd_moe_*`` in ``include/ragged_dot_hip.h``):

    routing = route(expert_ids, num_groups)                 # group_sizes, row_of_slot, slot_of_row
    x = dispatch(h, routing)                                # [tokens * top_k, d], rows sorted by expert
    y = ragged_dot(x, W, routing.group_sizes)               # the op itself
    out = combine(y, routing, weights)                      # [tokens, n]

``dispatch`` and ``combine`` are differentiable (each one's backward is the other kernel; the gradient of the combine
weights is ``rd_moe_combine_wgrad``).  torch supplies device memory and the stream, nothing else.
"""

from __future__ import annotations

from typing import NamedTuple, Optional

import torch

from . import _capi
from .ops import _DTYPES, _check_device, _stream_ptr

__all__ = ["Routing", "route", "dispatch", "combine"]


class Routing(NamedTuple):
    group_sizes: torch.Tensor   # int32 [g]      rows per expert
    row_of_slot: torch.Tensor   # int32 [tokens * top_k]  row of the sorted matrix each (token, choice) went to, -1 = dropped
    slot_of_row: torch.Tensor   # int32 [tokens * top_k]  inverse; -1 for rows past sum(group_sizes)
    tokens: int
    top_k: int


def route(expert_ids: torch.Tensor, num_groups: int) -> Routing:
    """Stable counting sort of the (token, choice) pairs by expert id.  ``expert_ids`` is integer ``[tokens, top_k]``;
    ids outside ``[0, num_groups)`` mark dropped pairs."""
    if expert_ids.dim() != 2:
        raise ValueError("expert_ids must be [tokens, top_k]")
    dev = _check_device(expert_ids)
    ids = expert_ids.to(torch.int32).contiguous()
    tokens, top_k = ids.shape
    slots = tokens * top_k
    group_sizes = torch.empty(num_groups, dtype=torch.int32, device=dev)
    row_of_slot = torch.empty(slots, dtype=torch.int32, device=dev)
    slot_of_row = torch.empty(slots, dtype=torch.int32, device=dev)
    ws_bytes = _capi.lib.rd_moe_route_workspace_bytes(tokens, top_k, num_groups)
    ws = torch.empty(max(ws_bytes, 256), dtype=torch.uint8, device=dev)
    with torch.cuda.device(dev):
        _capi.check(_capi.lib.rd_moe_route(_stream_ptr(dev), ids.data_ptr(), tokens, top_k, num_groups,
                                           group_sizes.data_ptr(), row_of_slot.data_ptr(), slot_of_row.data_ptr(),
                                           ws.data_ptr(), ws.numel()))
    return Routing(group_sizes, row_of_slot, slot_of_row, tokens, top_k)


def _dtype(t: torch.Tensor) -> int:
    if t.dtype not in _DTYPES or t.dtype == torch.float8_e4m3fn:
        raise TypeError(f"unsupported dtype {t.dtype}; rows are bfloat16, float16 or float32")
    return _DTYPES[t.dtype]


def _dispatch(h, r: Routing, row_scale):
    dev = _check_device(h, r.slot_of_row)
    h = h.contiguous()
    if h.dim() != 2 or h.shape[0] != r.tokens:
        raise ValueError(f"h must be [{r.tokens}, d]")
    d = h.shape[1]
    x = torch.empty((r.tokens * r.top_k, d), dtype=h.dtype, device=dev)
    with torch.cuda.device(dev):
        _capi.check(_capi.lib.rd_moe_dispatch(_stream_ptr(dev), h.data_ptr(), r.row_of_slot.data_ptr(), r.slot_of_row.data_ptr(),
                                              row_scale.data_ptr() if row_scale is not None else None, x.data_ptr(),
                                              r.tokens, r.top_k, d, _dtype(h)))
    return x


def _combine(y, r: Routing, weights):
    dev = _check_device(y, r.row_of_slot)
    y = y.contiguous()
    if y.dim() != 2 or y.shape[0] != r.tokens * r.top_k:
        raise ValueError(f"y must be [{r.tokens * r.top_k}, d]")
    d = y.shape[1]
    out = torch.empty((r.tokens, d), dtype=y.dtype, device=dev)
    with torch.cuda.device(dev):
        _capi.check(_capi.lib.rd_moe_combine(_stream_ptr(dev), y.data_ptr(), r.row_of_slot.data_ptr(),
                                             weights.data_ptr() if weights is not None else None, out.data_ptr(),
                                             r.tokens, r.top_k, d, _dtype(y)))
    return out


def _combine_wgrad(y, dout, r: Routing):
    dev = _check_device(y, dout)
    y, dout = y.contiguous(), dout.contiguous()
    dw = torch.empty(r.tokens * r.top_k, dtype=torch.float32, device=dev)
    with torch.cuda.device(dev):
        _capi.check(_capi.lib.rd_moe_combine_wgrad(_stream_ptr(dev), y.data_ptr(), dout.data_ptr(),
                                                   r.row_of_slot.data_ptr(), dw.data_ptr(), r.tokens, r.top_k,
                                                   y.shape[1], _dtype(y)))
    return dw


class _DispatchFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, h, routing):
        ctx.routing = routing
        return _dispatch(h, routing, None)

    @staticmethod
    def backward(ctx, dx):
        return _combine(dx, ctx.routing, None), None  # each token collects the gradients of its rows


class _CombineFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, y, weights, routing):
        ctx.routing = routing
        ctx.save_for_backward(y, weights)
        return _combine(y, routing, weights)

    @staticmethod
    def backward(ctx, dout):
        y, weights = ctx.saved_tensors
        r = ctx.routing
        dy = dw = None
        if ctx.needs_input_grad[0]:
            dy = _dispatch(dout, r, weights)  # dy[row] = weight of the row's slot * dout[token]
        if weights is not None and ctx.needs_input_grad[1]:
            dw = _combine_wgrad(y, dout, r)
        return dy, dw, None


def dispatch(h: torch.Tensor, routing: Routing) -> torch.Tensor:
    """``x[row] = h[token of row]``: ``[tokens, d] -> [tokens * top_k, d]`` sorted by expert; rows past
    ``sum(group_sizes)`` are zero."""
    return _DispatchFn.apply(h, routing)


def combine(y: torch.Tensor, routing: Routing, weights: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``out[token] = sum_choice weights[token, choice] * y[row of (token, choice)]`` with fp32 accumulation;
    ``weights`` is ``[tokens, top_k]`` (None = 1)."""
    slots = routing.tokens * routing.top_k
    w = None
    if weights is not None:
        w = weights.reshape(-1)
        if w.dtype != torch.float32 or not w.is_contiguous():
            w = w.to(torch.float32).contiguous()
        if w.numel() != slots:
            raise ValueError(f"weights must have {slots} entries")
    return _CombineFn.apply(y, w, routing)
