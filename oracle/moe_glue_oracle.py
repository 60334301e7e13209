"""CPU oracle for the token routing around ragged_dot.  TEST INFRASTRUCTURE ONLY.

The reference has no code for this step: its tests and tuner hand ragged_dot rows that are already sorted by group
(tests.py:51-71, tuning.py:41-47), i.e. the caller is expected to have done what this file states.  What is restated
here is therefore the textbook definition, written with numpy library routines that share nothing with the HIP
kernels:

* ``route``     - stable counting sort of the (token, slot) pairs by expert id: ``numpy.argsort(kind="stable")`` and
                  ``numpy.bincount``.  Pinned in tests/test_moe_glue.py by brute force on tiny inputs (a Python
                  loop that appends every slot to its expert's list), by the invariants sortedness / stability /
                  permutation-and-inverse, and by the committed fixture tests/golden/moe_route_golden.json.
* ``dispatch``  - a row gather (``numpy.take``), optionally scaled per row.
* ``combine``   - the weighted sum of each token's top_k rows, in float64 (the GPU sums in float32 in slot order; the
                  test tolerance is stated there).
* ``combine_wgrad`` - per (token, slot) dot products.
* ``dispatch``/``combine`` adjointness ``<dispatch(h), y> == <h, combine(y, w=1)>`` pins the pair against each other
  without any outside oracle.

Nothing in the shipped package may import this module.
"""

from __future__ import annotations

import numpy as np


def route(expert_ids: np.ndarray, g: int):
    """expert_ids: int32 [tokens, top_k] (or flat); ids outside [0, g) mark dropped slots.

    Returns (group_sizes[g], row_of_slot[S], slot_of_row[S]) as int32, S = tokens * top_k.  Kept slots are ordered by
    expert id, ties by slot index (stable); row_of_slot is -1 for dropped slots; slot_of_row is -1 for the rows past
    sum(group_sizes).
    """
    ids = np.asarray(expert_ids, dtype=np.int64).reshape(-1)
    S = ids.size
    keep = (ids >= 0) & (ids < g)
    group_sizes = np.bincount(ids[keep], minlength=g).astype(np.int32)
    order = np.argsort(np.where(keep, ids, g), kind="stable")  # dropped slots sort to the end
    total = int(keep.sum())
    slot_of_row = np.full(S, -1, dtype=np.int32)
    slot_of_row[:total] = order[:total]
    row_of_slot = np.full(S, -1, dtype=np.int32)
    row_of_slot[order[:total]] = np.arange(total, dtype=np.int32)
    return group_sizes, row_of_slot, slot_of_row


def dispatch(h: np.ndarray, slot_of_row: np.ndarray, top_k: int, row_scale: np.ndarray | None = None) -> np.ndarray:
    """x[row] = h[slot_of_row[row] // top_k] (times row_scale[slot] when given); rows with slot -1 are zero."""
    h = np.asarray(h, dtype=np.float32)
    S = slot_of_row.size
    x = np.zeros((S, h.shape[1]), dtype=np.float32)
    live = slot_of_row >= 0
    slots = slot_of_row[live].astype(np.int64)
    rows = np.take(h, slots // top_k, axis=0)
    if row_scale is not None:
        rows = rows * np.asarray(row_scale, dtype=np.float32).reshape(-1)[slots][:, None]
    x[live] = rows
    return x


def combine(y: np.ndarray, row_of_slot: np.ndarray, top_k: int, weights: np.ndarray | None = None) -> np.ndarray:
    """out[t] = sum_s weights[t, s] * y[row_of_slot[t * top_k + s]] over the kept slots (weights None = 1)."""
    y = np.asarray(y, dtype=np.float64)
    S = row_of_slot.size
    tokens = S // top_k
    w = np.ones(S) if weights is None else np.asarray(weights, dtype=np.float64).reshape(-1)
    out = np.zeros((tokens, y.shape[1]), dtype=np.float64)
    for s in range(top_k):
        rows = row_of_slot.reshape(tokens, top_k)[:, s]
        live = rows >= 0
        out[live] += w.reshape(tokens, top_k)[live, s][:, None] * y[rows[live]]
    return out


def combine_wgrad(y: np.ndarray, dout: np.ndarray, row_of_slot: np.ndarray, top_k: int) -> np.ndarray:
    """dw[t, s] = <y[row_of_slot[t * top_k + s]], dout[t]>; zero for dropped slots."""
    y = np.asarray(y, dtype=np.float64)
    dout = np.asarray(dout, dtype=np.float64)
    tokens = dout.shape[0]
    rows = row_of_slot.reshape(tokens, top_k)
    dw = np.zeros((tokens, top_k), dtype=np.float64)
    for s in range(top_k):
        live = rows[:, s] >= 0
        dw[live, s] = np.einsum("td,td->t", y[rows[live, s]], dout[live])
    return dw
