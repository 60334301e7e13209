"""ctypes binding of ``csrc/libragged_dot_hip.so`` (the C ABI declared in ``include/ragged_dot_hip.h``).

The library is built in-tree by ``make -C gpu_ragged_dot_amd/csrc`` (or ``__graft_entry__.build()``).  There is no
fallback: if the shared object is missing, importing this module raises.
"""

from __future__ import annotations

import ctypes
import os

try:  # loaded first, when present, so that the HIP runtime already in the process is the one the library binds to
    import torch  # noqa: F401
except ImportError:  # a JAX-only process: the library then loads the system HIP runtime, as jaxlib's ROCm plugin does
    torch = None

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "csrc", "libragged_dot_hip.so")

RD_DTYPE_BF16 = 0
RD_DTYPE_F32 = 1
RD_DTYPE_F32_BF16 = 2  # float32 arrays rounded to bfloat16 for the bf16 matrix cores (compute_dtype=bfloat16)
RD_DTYPE_F8E4M3_BF16 = 3  # float8 e4m3fn operands widened to bfloat16 for the bf16 matrix cores, bfloat16 out
RD_DTYPE_F16 = 4  # float16 arrays on the float16 matrix-core instruction, fp32 accumulation, float16 out

RD_OK = 0
RD_ERR_INVALID_ARGUMENT = -1
RD_ERR_UNSUPPORTED = -2
RD_ERR_WORKSPACE = -3
RD_ERR_HIP = -4

OP_GMM, OP_GMM_TRANS, OP_TGMM = 0, 1, 2


class RaggedDotError(RuntimeError):
    """A call into the HIP library returned a non-zero status."""

    def __init__(self, status: int, message: str):
        super().__init__(f"ragged_dot_hip status {status}: {message}")
        self.status = status


class VariantInfo(ctypes.Structure):
    _fields_ = [
        ("id", ctypes.c_int),
        ("tile_m", ctypes.c_int),
        ("tile_n", ctypes.c_int),
        ("tile_k", ctypes.c_int),
        ("waves_m", ctypes.c_int),
        ("waves_n", ctypes.c_int),
        ("vec", ctypes.c_int),
        ("dtype", ctypes.c_int),
        ("direct_to_lds", ctypes.c_int),
        ("stages", ctypes.c_int),
        ("name", ctypes.c_char * 48),
    ]


RD_DECODE_ROWS = -1  # Plan.decode_nb: whole-row slices
ABI_VERSION = 3  # RD_ABI_VERSION of include/ragged_dot_hip.h this file mirrors


class Plan(ctypes.Structure):
    _fields_ = [("variant", ctypes.c_int), ("group_m", ctypes.c_int), ("group_n", ctypes.c_int),
                ("decode_nb", ctypes.c_int), ("split_k", ctypes.c_int)]

    def __init__(self, variant=-1, group_m=0, decode_nb=0, group_n=0, split_k=0):
        super().__init__(variant, group_m, group_n, decode_nb, split_k)

    def __repr__(self):
        return (f"Plan(variant={self.variant}, group_m={self.group_m}, group_n={self.group_n}, "
                f"decode_nb={self.decode_nb}, split_k={self.split_k})")


# every symbol the header declares; checked at load time
EXPORTS = (
    "rd_abi_version",
    "rd_last_error",
    "rd_num_variants",
    "rd_get_variant",
    "rd_default_plan",
    "rd_sched_map",
    "rd_sched_map_len",
    "rd_gmm_workspace_bytes",
    "rd_gmm",
    "rd_gmm_sharded",
    "rd_tgmm_sharded",
    "rd_gmm_noalloc_scratch_bytes",
    "rd_gmm_noalloc",
    "rd_tgmm_workspace_bytes",
    "rd_tgmm",
    "rd_probe_stream_read",
    "rd_moe_route_workspace_bytes",
    "rd_moe_route",
    "rd_moe_dispatch",
    "rd_moe_combine",
    "rd_moe_combine_wgrad",
)


def _load() -> ctypes.CDLL:
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `make -C {os.path.dirname(LIB_PATH)} -j8` "
            "(hipcc --offload-arch=gfx950).  There is no CPU or PyTorch fallback for these ops."
        )
    lib = ctypes.CDLL(LIB_PATH)
    for name in EXPORTS:
        if not hasattr(lib, name):
            raise ImportError(f"{LIB_PATH} does not export {name}")
    vp, ip, i, sz = ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t
    lib.rd_abi_version.restype = i
    if lib.rd_abi_version() != ABI_VERSION:
        raise ImportError(f"{LIB_PATH} has ABI version {lib.rd_abi_version()}, this binding is for {ABI_VERSION}: rebuild it")
    lib.rd_last_error.restype = ctypes.c_char_p
    lib.rd_num_variants.restype = i
    lib.rd_get_variant.argtypes = [i, ctypes.POINTER(VariantInfo)]
    lib.rd_get_variant.restype = i
    lib.rd_default_plan.argtypes = [i, i, i, i, i, i, ctypes.POINTER(Plan)]
    lib.rd_default_plan.restype = i
    lib.rd_sched_map.argtypes = [vp, ip, i, i, i, ip, ip, ip, ip]
    lib.rd_sched_map.restype = i
    lib.rd_sched_map_len.argtypes = [i, i, i]
    lib.rd_sched_map_len.restype = i
    lib.rd_gmm_workspace_bytes.argtypes = [i, i, ctypes.POINTER(Plan)]
    lib.rd_gmm_workspace_bytes.restype = sz
    lib.rd_gmm.argtypes = [vp, vp, vp, ip, vp, i, i, i, i, i, i, ctypes.POINTER(Plan), vp, sz]
    lib.rd_gmm.restype = i
    lib.rd_gmm_sharded.argtypes = [vp, vp, vp, ip, vp, i, i, i, i, i, i, i, i, ctypes.POINTER(Plan), vp, sz]
    lib.rd_gmm_sharded.restype = i
    lib.rd_tgmm_sharded.argtypes = [vp, vp, vp, ip, vp, i, i, i, i, i, i, i, ctypes.POINTER(Plan), vp, sz]
    lib.rd_tgmm_sharded.restype = i
    lib.rd_gmm_noalloc_scratch_bytes.argtypes = []
    lib.rd_gmm_noalloc_scratch_bytes.restype = sz
    lib.rd_gmm_noalloc.argtypes = [vp, vp, vp, ip, vp, i, i, i, i, i, i, ctypes.POINTER(Plan)]
    lib.rd_gmm_noalloc.restype = i
    lib.rd_tgmm_workspace_bytes.argtypes = [i, i, ctypes.POINTER(Plan)]
    lib.rd_tgmm_workspace_bytes.restype = sz
    lib.rd_tgmm.argtypes = [vp, vp, vp, ip, vp, i, i, i, i, i, ctypes.POINTER(Plan), vp, sz]
    lib.rd_tgmm.restype = i
    lib.rd_probe_stream_read.argtypes = [vp, vp, sz, sz, vp]
    lib.rd_probe_stream_read.restype = i
    lib.rd_moe_route_workspace_bytes.argtypes = [i, i, i]
    lib.rd_moe_route_workspace_bytes.restype = sz
    lib.rd_moe_route.argtypes = [vp, ip, i, i, i, ip, ip, ip, vp, sz]
    lib.rd_moe_route.restype = i
    lib.rd_moe_dispatch.argtypes = [vp, vp, ip, ip, vp, vp, i, i, i, i]
    lib.rd_moe_dispatch.restype = i
    lib.rd_moe_combine.argtypes = [vp, vp, ip, vp, vp, i, i, i, i]
    lib.rd_moe_combine.restype = i
    lib.rd_moe_combine_wgrad.argtypes = [vp, vp, vp, ip, vp, i, i, i, i]
    lib.rd_moe_combine_wgrad.restype = i
    return lib


lib = _load()


def check(status: int) -> None:
    if status != RD_OK:
        raise RaggedDotError(status, (lib.rd_last_error() or b"").decode("utf-8", "replace"))


def variants() -> list[VariantInfo]:
    out = []
    for idx in range(lib.rd_num_variants()):
        info = VariantInfo()
        check(lib.rd_get_variant(idx, ctypes.byref(info)))
        out.append(info)
    return out


def default_plan(op: int, m: int, k: int, n: int, g: int, dtype: int = RD_DTYPE_BF16) -> Plan:
    plan = Plan()
    check(lib.rd_default_plan(op, m, k, n, g, dtype, ctypes.byref(plan)))
    return plan
