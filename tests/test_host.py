"""CPU-side checks of the host layer: the C ABI library loads and exports every symbol the header declares, argument
validation returns error codes (no device work is launched), and the planner follows the reference's block rules."""

import ctypes
import os
import re

import pytest
import torch

from gpu_ragged_dot_amd import _capi, planner
from oracle import ragged_dot_oracle as oracle

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_functions():
    text = open(os.path.join(ROOT, "include", "ragged_dot_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(rd_[a-z_0-9]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = _declared_functions()
    assert len(names) >= 11
    lib = ctypes.CDLL(_capi.LIB_PATH)
    for name in names:
        assert hasattr(lib, name), f"{name} declared in include/ragged_dot_hip.h but not exported"
    assert sorted(_capi.EXPORTS) == names, "the ctypes binding must cover exactly what the header declares"
    assert _capi.lib.rd_abi_version() == 3


def test_variant_table():
    vs = _capi.variants()
    assert len(vs) >= 2
    names = [v.name.decode() for v in vs]
    assert len(set(names)) == len(names)
    assert any(v.vec == 0 and v.dtype == _capi.RD_DTYPE_BF16 for v in vs), "an any-shape bf16 variant must exist"
    assert any(v.dtype == _capi.RD_DTYPE_F32 for v in vs), "float32 operands need a kernel too"
    for v in vs:
        assert v.tile_m % (32 * v.waves_m) == 0 and v.tile_n % (32 * v.waves_n) == 0 and v.tile_k % 16 == 0
        if v.direct_to_lds:
            elem = 1 if v.dtype == _capi.RD_DTYPE_F8E4M3_BF16 else 2  # bytes per operand element in the LDS ring
            assert v.vec == 1 and v.stages * (v.tile_m + v.tile_n) * v.tile_k * elem <= 160 * 1024


def test_argument_validation_returns_codes():
    lib = _capi.lib
    one = ctypes.c_void_p(16)  # never dereferenced: validation fails first
    rc = lib.rd_gmm(None, one, one, one, one, 8, 8, 8, 0, 0, _capi.RD_DTYPE_BF16, None, one, 1 << 20)
    assert rc == _capi.RD_ERR_INVALID_ARGUMENT and b"g=0" in lib.rd_last_error()
    rc = lib.rd_gmm(None, one, one, one, one, -1, 8, 8, 2, 0, _capi.RD_DTYPE_BF16, None, one, 1 << 20)
    assert rc == _capi.RD_ERR_INVALID_ARGUMENT
    rc = lib.rd_gmm(None, one, one, None, one, 8, 8, 8, 2, 0, _capi.RD_DTYPE_BF16, None, one, 1 << 20)
    assert rc == _capi.RD_ERR_INVALID_ARGUMENT and b"null" in lib.rd_last_error()
    rc = lib.rd_gmm(None, one, one, one, one, 8, 8, 8, 2, 0, 7, None, one, 1 << 20)
    assert rc == _capi.RD_ERR_INVALID_ARGUMENT
    bf16_id = next(v.id for v in _capi.variants() if v.dtype == _capi.RD_DTYPE_BF16 and not v.vec)
    plan = _capi.Plan(bf16_id, 0, 0)  # a bf16 variant cannot take float32 operands (checked before any launch)
    rc = lib.rd_gmm(None, one, one, one, one, 8, 8, 8, 2, 0, _capi.RD_DTYPE_F32, ctypes.byref(plan), one, 1 << 20)
    assert rc == _capi.RD_ERR_UNSUPPORTED
    rc = lib.rd_tgmm(None, one, one, one, one, 8, 8, 8, 0, _capi.RD_DTYPE_BF16, None, one, 1 << 20)
    assert rc == _capi.RD_ERR_INVALID_ARGUMENT
    rc = lib.rd_sched_map(None, one, 0, 8, 8, one, one, one, one)
    assert rc == _capi.RD_ERR_INVALID_ARGUMENT
    rc = lib.rd_sched_map(None, one, 4, 8, 0, one, one, one, one)
    assert rc == _capi.RD_ERR_INVALID_ARGUMENT
    with pytest.raises(_capi.RaggedDotError):
        _capi.check(rc)
    assert lib.rd_get_variant(10 ** 6, ctypes.byref(_capi.VariantInfo())) == _capi.RD_ERR_INVALID_ARGUMENT
    # a plan that names a missing variant, a too-small workspace, a vector variant on an unaligned shape
    plan = _capi.Plan(10 ** 6, 0, 0)
    rc = lib.rd_gmm(None, one, one, one, one, 8, 8, 8, 2, 0, _capi.RD_DTYPE_BF16, ctypes.byref(plan), one, 1 << 20)
    assert rc == _capi.RD_ERR_INVALID_ARGUMENT
    rc = lib.rd_gmm(None, one, one, one, one, 64, 64, 64, 2, 0, _capi.RD_DTYPE_BF16, None, one, 8)
    assert rc == _capi.RD_ERR_WORKSPACE
    vec_id = next(v.id for v in _capi.variants() if v.vec and v.dtype == _capi.RD_DTYPE_BF16)
    plan = _capi.Plan(vec_id, 0, 0)
    rc = lib.rd_gmm(None, one, one, one, one, 64, 58, 77, 2, 0, _capi.RD_DTYPE_BF16, ctypes.byref(plan), one, 1 << 20)
    assert rc == _capi.RD_ERR_UNSUPPORTED


def test_workspace_and_map_sizes():
    lib = _capi.lib
    assert lib.rd_sched_map_len(16384, 8, 512) == 40  # U of the Mixtral config at the reference's chunk
    assert lib.rd_sched_map_len(64, 128, 512) == 129
    assert lib.rd_sched_map_len(0, 3, 8) == 3
    for m, g in ((16384, 8), (32768, 256), (64, 128), (0, 1)):
        need = lib.rd_gmm_workspace_bytes(m, g, None)
        for v in _capi.variants():
            U = -(-m // v.tile_m) + g
            assert need >= (g + 2 * U + 1) * 4
        assert lib.rd_tgmm_workspace_bytes(m, g, None) >= (g + 2 * (g + 1) + 1) * 4
        # the K-split of the last round needs 256 slots of tile_m x tile_n fp32 on top of the map; split_k = -1 and
        # variants without it only need the map
        import ctypes
        whole = lib.rd_gmm_workspace_bytes(m, g, ctypes.byref(_capi.Plan(-1, split_k=-1)))
        assert whole < (1 << 20) and need >= whole
        for v in _capi.variants():
            split = lib.rd_gmm_workspace_bytes(m, g, ctypes.byref(_capi.Plan(v.id)))
            extra = 256 * 4 + 256 * v.tile_m * v.tile_n * 4
            assert split in (whole, whole + extra), (v.name, split, whole)
            if v.direct_to_lds and v.dtype in (_capi.RD_DTYPE_BF16, _capi.RD_DTYPE_F8E4M3_BF16):
                assert split == whole + extra and need >= split


def test_planner_block_rules_match_the_oracle():
    for args in ((64, 64, 64, 16384, 4096, 14336), (16, 16, 16, 171, 58, 77), (8, 8, 8, 100, 100, 100),
                 (256, 256, 256, 5, 40, 9), (32, 64, 16, 128, 512, 64)):
        assert planner.normalize_gmm_blocks(*args) == oracle.gmm_block_sizes(*args)
        assert planner.normalize_tgmm_blocks(*args) == oracle.tgmm_block_sizes(*args)


def test_planner_choices():
    vs = {v.id: v for v in _capi.variants()}
    p = planner.select_plan(_capi.OP_GMM, 171, 58, 77, 8)
    assert vs[p.variant].vec == 0 and p.decode_nb == 0  # odd pitches -> any-shape variant
    p = planner.select_plan(_capi.OP_TGMM, 171, 58, 77, 8, dtype=_capi.RD_DTYPE_F32)
    assert vs[p.variant].dtype == _capi.RD_DTYPE_F32
    p = planner.select_plan(_capi.OP_GMM, 64, 2048, 768, 128)
    assert p.decode_nb == _capi.RD_DECODE_ROWS  # a few rows per expert -> streaming kernel (whole-row slices)
    p = planner.select_plan(_capi.OP_GMM_TRANS, 64, 2048, 768, 128)
    assert p.decode_nb == _capi.RD_DECODE_ROWS  # weights stored [g, n, k] have a streaming kernel of their own
    p = planner.select_plan(_capi.OP_GMM_TRANS, 64, 16384, 768, 128)
    assert p.decode_nb == 0  # ... up to the contraction length whose activations it can stage
    p = planner.select_plan(_capi.OP_GMM, 512, 2048, 768, 128)
    assert p.decode_nb == _capi.RD_DECODE_ROWS  # four rows per expert on average: still one pass of up to eight
    p = planner.select_plan(_capi.OP_GMM, 1024, 2048, 768, 128)
    assert p.decode_nb == 0
    p = planner.select_plan(_capi.OP_GMM, 256, 7168, 2048, 256)
    assert p.decode_nb == 0  # enough 256-column tiles for the tile kernels' streaming routines
    p = planner.select_plan(_capi.OP_GMM, 64, 7168, 2048, 256)
    assert p.decode_nb == _capi.RD_DECODE_ROWS
    # float8: the streaming kernel for weights stored [g, n, k] only, up to one row per group on average
    f8 = _capi.RD_DTYPE_F8E4M3_BF16
    assert planner.select_plan(_capi.OP_GMM_TRANS, 64, 2048, 768, 128, dtype=f8).decode_nb == _capi.RD_DECODE_ROWS
    assert planner.select_plan(_capi.OP_GMM_TRANS, 128, 2048, 768, 128, dtype=f8).decode_nb == _capi.RD_DECODE_ROWS
    assert planner.select_plan(_capi.OP_GMM_TRANS, 256, 2048, 768, 128, dtype=f8).decode_nb == 0
    assert planner.select_plan(_capi.OP_GMM_TRANS, 64, 2056, 768, 128, dtype=f8).decode_nb == 0  # k % 16
    assert planner.select_plan(_capi.OP_GMM, 64, 2048, 768, 128, dtype=f8).decode_nb == 0
    assert planner.select_plan(_capi.OP_GMM_TRANS, 64, 2048, 768, 128, dtype=_capi.RD_DTYPE_F32).decode_nb == 0
    p = planner.select_plan(_capi.OP_GMM, 16384, 4096, 14336, 8)
    assert vs[p.variant].tile_m == 256 and vs[p.variant].tile_n == 256
    p = planner.select_plan(_capi.OP_GMM, 16384, 4096, 14336, 8, block_m=128, block_k=64, block_n=128)
    assert (vs[p.variant].tile_m, vs[p.variant].tile_n) == (128, 128)  # explicit request -> nearest compiled shape


def test_default_plan_scales_the_tile_with_the_problem():
    """The library's shape-only default (no tuned-table entry): 256 x 256 cores for many rounds of tiles or a long
    contraction, the 128-row cores when those would leave compute units idle, register-staged tiles for small outputs;
    all three products; float32 picks its larger tile only when the output fills the device with it."""
    vs = {v.id: v for v in _capi.variants()}
    tile = lambda op, m, k, n, g, **kw: (lambda v: (v.tile_m, v.tile_n))(vs[_capi.default_plan(op, m, k, n, g, **kw).variant])
    for op in (_capi.OP_GMM, _capi.OP_GMM_TRANS, _capi.OP_TGMM):
        assert tile(op, 16384, 4096, 14336, 8) == (256, 256)
        assert tile(op, 32768, 7168, 2048, 256) == (256, 256)
    assert tile(_capi.OP_GMM, 6144, 6144, 1536, 6) == (256, 256)      # few tiles, long contraction
    assert tile(_capi.OP_GMM, 65536, 512, 512, 64) == (128, 256)      # short contraction: two work-groups per compute unit hide the tile set-up
    assert tile(_capi.OP_GMM_TRANS, 8192, 4096, 256, 16) == (64, 64)      # 144 tiles of 128 x 128: too few
    assert tile(_capi.OP_TGMM, 4096, 1024, 1024, 8) == (128, 128)
    assert max(tile(_capi.OP_GMM, 2048, 4096, 512, 4)) <= 128 and max(tile(_capi.OP_GMM, 256, 64, 64, 4)) <= 128
    # few 128 x 128 tiles and a moderate contraction: four times as many 64 x 64 tiles, walked in blocks of 16
    assert tile(_capi.OP_GMM, 256, 4096, 4096, 2) == (64, 64) and tile(_capi.OP_GMM, 1280, 1280, 1280, 10) == (64, 64)
    p = _capi.default_plan(_capi.OP_GMM_TRANS, 1024, 2048, 512, 4)
    assert (vs[p.variant].tile_m, vs[p.variant].tile_n, p.group_m, p.group_n) == (64, 64, 4, 4)
    assert tile(_capi.OP_GMM_TRANS, 1536, 8192, 1024, 3) == (128, 128)   # ... but not with a contraction of 8192
    # trans_rhs, long contraction, under a round of 256 x 256 tiles: the eight-wave 256 x 256 core and its K-split
    assert vs[_capi.default_plan(_capi.OP_GMM_TRANS, 512, 8192, 8192, 1).variant].name.decode() == "p256x256x32_w2x4_s4"
    name = lambda op, m, k, n, g: vs[_capi.default_plan(op, m, k, n, g).variant].name.decode()
    # forward product, few tiles: the four-wave core for long groups, the eight-wave per-operand-ring one for groups of a tile's height
    assert name(_capi.OP_GMM, 6144, 6144, 1536, 6) == "w256x256x32_w2x2_s5" and name(_capi.OP_GMM, 1792, 7168, 7168, 7) == "q256x256x32_w2x4"
    # tgmm with groups far shorter than a tile: three 128 x 128 work-groups per compute unit (not at the DeepSeek-V3 size)
    assert tile(_capi.OP_TGMM, 3072, 3072, 3072, 48) == (128, 128) and tile(_capi.OP_TGMM, 4096, 7168, 2048, 64) == (128, 128)
    assert tile(_capi.OP_TGMM, 16384, 2048, 4096, 128) == (256, 256)
    assert tile(_capi.OP_GMM, 8192, 4096, 4096, 8, dtype=_capi.RD_DTYPE_F32) == (128, 128)
    assert tile(_capi.OP_GMM, 512, 256, 256, 4, dtype=_capi.RD_DTYPE_F32) == (64, 64)


def test_cpu_tensors_are_rejected_loudly():
    import gpu_ragged_dot_amd as rd

    x = torch.zeros(8, 8, dtype=torch.bfloat16)
    A = torch.zeros(2, 8, 8, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="no CPU path"):
        rd.ragged_dot(x, A, torch.tensor([4, 4], dtype=torch.int32))
    with pytest.raises(NotImplementedError):
        rd.ragged_dot(x, A, torch.tensor([4, 4], dtype=torch.int32), interpret=True)
    with pytest.raises(AssertionError):
        rd.ragged_dot(x, A[0], torch.tensor([4, 4], dtype=torch.int32))  # gpu_ragged_dot.py:188
    with pytest.raises(AssertionError):
        rd.ragged_dot(x, A, torch.tensor([4, 2, 2], dtype=torch.int32))  # gpu_ragged_dot.py:189
    with pytest.raises(AssertionError):
        rd.tgmm(x, torch.zeros(9, 8, dtype=torch.bfloat16), torch.tensor([4, 4], dtype=torch.int32))  # :304


def test_committed_traffic_figures_belong_to_the_plans_in_use():
    """profiles/hbm_traffic.json tags every counter-derived figure with the plan it was measured under; bench.py drops a
    figure whose tag is not the plan in use.  Keep the committed table in step with the planner."""
    import json
    import os

    import bench
    from gpu_ragged_dot_amd import workloads

    with open(os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "profiles", "hbm_traffic.json")) as f:
        table = json.load(f)
    for name, kernels in table.items():
        if name.startswith("_"):
            continue
        w = workloads.WORKLOADS[name]
        dims = {"fwd": (0, w.m, w.k, w.n), "dlhs": (1, w.m, w.n, w.k), "drhs": (2, w.m, w.k, w.n)}
        for kernel, entry in kernels.items():
            op, m, k, n = dims[kernel]
            assert entry["bytes"] > 0
            assert entry["plan"] == bench._plan_text(planner.select_plan(op, m, k, n, w.g), planner), (name, kernel)
