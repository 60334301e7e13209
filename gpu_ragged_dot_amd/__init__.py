"""MI355X-native ragged (grouped) matrix products with the Python surface of ``gpu_ragged_dot``.

``ragged_dot(x[m,k], A[g,k,n], group_sizes[g], ...)`` and ``trans_ragged_dot(x[m,k], y[m,n], group_sizes[g], ...)``
(gpu_ragged_dot.py:30, 406, 454) computed by hand-written gfx950 kernels behind a C ABI.
"""

from .planner import CHUNK_M, DEFAULT_BLOCK_K, DEFAULT_BLOCK_M, DEFAULT_BLOCK_N

try:
    import torch as _torch  # noqa: F401
except ImportError:  # a JAX-only process: the same names live in gpu_ragged_dot_amd.jax_adapter
    _torch = None
if _torch is not None:
    from . import moe  # noqa: F401  (route / dispatch / combine around ragged_dot)
    from .ops import gmm, make_group_metadata, ragged_dot, ragged_dot_vjp, tgmm, trans_ragged_dot

__all__ = ["gmm", "tgmm", "ragged_dot", "trans_ragged_dot", "ragged_dot_vjp", "make_group_metadata",
           "moe", "CHUNK_M", "DEFAULT_BLOCK_M", "DEFAULT_BLOCK_N", "DEFAULT_BLOCK_K"]
