"""Pins the CPU oracle (oracle/ragged_dot_oracle.py) without importing the reference or JAX: hand-computed known
answers, closed forms, special cases that reduce to independent library routines, adjoint identities, and the
reference's own all-ones known-answer case (tests.py:67,103)."""

import numpy as np
import pytest

from oracle import ragged_dot_oracle as oracle
from tests import util


# ---- bf16 rounding ---------------------------------------------------------------------------------------------------

def test_bf16_round_to_nearest_even_known_values():
    f = lambda bits: np.array([bits], dtype=np.uint32).view(np.float32)
    # 1.0 = 0x3F800000; one bf16 ulp above is 0x3F810000.  Ties go to the even mantissa.
    assert oracle.f32_to_bf16_bits(f(0x3F800000))[0] == 0x3F80
    assert oracle.f32_to_bf16_bits(f(0x3F808000))[0] == 0x3F80  # exactly half-way, low bit 0 -> stays
    assert oracle.f32_to_bf16_bits(f(0x3F818000))[0] == 0x3F82  # half-way, low bit 1 -> rounds up to even
    assert oracle.f32_to_bf16_bits(f(0x3F808001))[0] == 0x3F81  # just above half-way
    assert oracle.f32_to_bf16_bits(f(0x7F800000))[0] == 0x7F80  # +inf
    assert oracle.f32_to_bf16_bits(f(0x7F7FFFFF))[0] == 0x7F80  # max float rounds to inf
    nan = oracle.f32_to_bf16_bits(f(0x7FC00001))[0]
    assert (nan & 0x7F80) == 0x7F80 and (nan & 0x007F) != 0


def test_bf16_matches_torch():
    import torch

    a = np.random.default_rng(0).normal(size=10000).astype(np.float32) * 100
    ours = oracle.round_to(a, "bfloat16")
    theirs = torch.from_numpy(a).to(torch.bfloat16).float().numpy()
    np.testing.assert_array_equal(ours, theirs)


def test_float16_round_to_nearest_even_known_values():
    """round_to(.., 'float16'): IEEE half, 10 mantissa bits, ties to even, overflow to infinity, subnormals down to 2^-24."""
    r = lambda v: float(oracle.round_to(np.array([v], np.float32), "float16")[0])
    assert r(1.0 + 2.0 ** -11) == 1.0                       # half-way between 1 and 1 + 2^-10, even mantissa below
    assert r(1.0 + 3 * 2.0 ** -11) == 1.0 + 2.0 ** -9       # half-way, odd mantissa below: up to the even one
    assert r(1.0 + 2.0 ** -11 + 2.0 ** -20) == 1.0 + 2.0 ** -10   # just above half-way
    assert r(65504.0) == 65504.0 and r(65519.0) == 65504.0 and np.isinf(r(65520.0))   # largest value; the tie goes to inf
    assert r(2.0 ** -24) == 2.0 ** -24 and r(2.0 ** -25) == 0.0 and r(1.5 * 2.0 ** -24) == 2.0 ** -23   # subnormals, ties to even
    assert r(-0.1) == -r(0.1) and abs(r(0.1) - 0.1) <= 2.0 ** -14


def test_float16_matches_torch():
    import torch

    a = np.random.default_rng(1).normal(size=10000).astype(np.float32) * 300
    a[:4] = [7e4, -7e4, 1e-7, 6e-8]
    ours = oracle.round_to(a, "float16")
    theirs = torch.from_numpy(a).to(torch.float16).float().numpy()
    np.testing.assert_array_equal(ours, theirs)


# ---- scheduling map (gpu_ragged_dot.py:70-90) -------------------------------------------------------------------------

def test_metadata_hand_computed():
    # sizes [3, 0, 5], chunk 2, m 8: tiles per group [2, 0, 3]; U = 4 + 3 = 7
    md = oracle.make_gmm_group_metadata(np.array([3, 0, 5], np.int32), 8, 2)
    assert md.group_offsets.tolist() == [0, 3, 3]
    assert md.row_it2group.tolist() == [0, 0, 2, 2, 2, 0, 0]
    assert md.row_it2it_in_group.tolist() == [0, 1, 0, 1, 2, 0, 0]
    assert int(md.total_row_its) == 5
    # one chunk per group, rows left over: sizes [4, 1], chunk 512, m 10 -> U = 1 + 2
    md = oracle.make_gmm_group_metadata(np.array([4, 1], np.int32), 10, 512)
    assert md.row_it2group.tolist() == [0, 1, 0]
    assert md.row_it2it_in_group.tolist() == [0, 0, 0]
    assert md.group_offsets.tolist() == [0, 4] and int(md.total_row_its) == 2


def _closed_form(gs, m, c):
    g = gs.size
    bpg = (gs + c - 1) // c
    U = (m + c - 1) // c + g
    t2g = np.repeat(np.arange(g, dtype=np.int32), bpg)
    t2it = np.concatenate([np.arange(b, dtype=np.int32) for b in bpg] + [np.zeros(0, np.int32)])
    pad = lambda a: np.concatenate([a, np.zeros(U - a.size, np.int32)])[:U]
    return np.cumsum(gs) - gs, pad(t2g), pad(t2it), int(bpg.sum())


@pytest.mark.parametrize("seed", range(30))
def test_metadata_closed_form_and_invariants(seed):
    rng = np.random.default_rng(seed)
    g = int(rng.integers(1, 70))
    m = int(rng.integers(1, 5000))
    c = int(rng.choice([1, 3, 8, 64, 512]))
    gs = oracle.generate_group_sizes(seed, g, int(m * rng.choice([1.0, 0.7, 0.5, 0.0])))
    gs[rng.random(g) < 0.25] = 0
    md = oracle.make_gmm_group_metadata(gs, m, c)
    offs, t2g, t2it, total = _closed_form(gs, m, c)
    np.testing.assert_array_equal(md.group_offsets, offs)
    np.testing.assert_array_equal(md.row_it2group, t2g)
    np.testing.assert_array_equal(md.row_it2it_in_group, t2it)
    assert int(md.total_row_its) == total
    # invariants: enough slots; groups ascend over the used range; chunk index restarts at 0 and steps by 1;
    # every row of every non-empty group is covered exactly once by (group, chunk) pairs
    U = md.row_it2group.size
    assert total <= U
    used_g, used_it = md.row_it2group[:total], md.row_it2it_in_group[:total]
    assert np.all(np.diff(used_g) >= 0)
    assert np.all(gs[used_g] > 0)
    if total > 0:
        starts = np.r_[True, np.diff(used_g) != 0]
        assert np.all(used_it[starts] == 0) and np.all(np.diff(used_it)[~starts[1:]] == 1)
    covered = np.zeros(int(gs.sum()), np.int32)
    for gi, it in zip(used_g, used_it):
        lo = offs[gi] + it * c
        covered[lo:min(lo + c, offs[gi] + gs[gi])] += 1
    assert np.all(covered == 1)
    assert not np.any(md.row_it2group[total:]) and not np.any(md.row_it2it_in_group[total:])


def test_metadata_dtypes_are_int32():
    md = oracle.make_gmm_group_metadata(np.array([5, 6], np.int64), 11, 4)
    for a in md:
        assert np.asarray(a).dtype == np.int32


# ---- host planning rules (gpu_ragged_dot.py:194-197, 308-314, 212-213, 326) ----------------------------------------

def test_block_rules_table():
    assert oracle.gmm_block_sizes(64, 64, 64, 16384, 4096, 14336) == (64, 64, 64)
    assert oracle.gmm_block_sizes(16, 16, 16, 171, 58, 77) == (16, 16, 16)
    assert oracle.gmm_block_sizes(64, 64, 64, 171, 58, 77) == (64, 64, 64)  # min(64,58)=58 -> 64
    assert oracle.gmm_block_sizes(8, 8, 8, 100, 100, 100) == (8, 16, 16)  # only k and n are raised to 16
    assert oracle.gmm_block_sizes(256, 256, 256, 5, 40, 9) == (8, 64, 16)
    assert oracle.tgmm_block_sizes(8, 8, 8, 100, 100, 100) == (16, 16, 16)  # all three raised
    assert oracle.tgmm_block_sizes(64, 64, 64, 171, 58, 77) == (64, 64, 64)
    assert oracle.tgmm_block_sizes(256, 256, 256, 5, 40, 9) == (16, 64, 16)
    assert [oracle.next_power_of_2(v) for v in (0, 1, 2, 3, 58, 64, 65)] == [1, 1, 2, 4, 64, 64, 128]
    assert oracle.gmm_grid(16384, 14336, 8, 64, 512) == (40, 224)  # launch shapes quoted for the Mixtral config
    assert oracle.gmm_grid(64, 768, 128, 64, 512) == (129, 12)
    assert oracle.tgmm_grid(4096, 14336, 8, 64, 64) == (8, 64, 224)


# ---- definition: special cases that reduce to independent routines ----------------------------------------------------

def test_gmm_single_group_is_plain_matmul():
    rng = np.random.default_rng(1)
    x = rng.normal(size=(37, 20)).astype(np.float32)
    A = rng.normal(size=(1, 20, 11)).astype(np.float32)
    np.testing.assert_allclose(oracle.gmm(x, A, [37], out_dtype="float32"), x @ A[0], rtol=1e-6, atol=1e-6)
    y = oracle.gmm(x, A, [30], out_dtype="float32")
    np.testing.assert_allclose(y[:30], x[:30] @ A[0], rtol=1e-6, atol=1e-6)
    assert not np.any(y[30:])


def test_gmm_equal_groups_is_batched_matmul():
    rng = np.random.default_rng(2)
    g, r, k, n = 5, 7, 12, 9
    x = rng.normal(size=(g * r, k))
    A = rng.normal(size=(g, k, n))
    want = np.einsum("grk,gkn->grn", x.reshape(g, r, k), A).reshape(g * r, n)
    np.testing.assert_allclose(oracle.gmm(x, A, [r] * g, out_dtype="float32", acc=np.float64), want, rtol=1e-12)
    want_t = np.einsum("grk,grn->gkn", x.reshape(g, r, k), want.reshape(g, r, n))
    np.testing.assert_allclose(oracle.tgmm(x, want, [r] * g, out_dtype="float32", acc=np.float64), want_t, rtol=1e-12)


def test_all_ones_known_answer():
    """tests.py:67,103 random_inputs=False: every valid output of gmm is exactly k; tgmm gives the group size."""
    gs = np.array([3, 0, 10, 4], np.int32)
    x, A, dy = np.ones((20, 58), np.float32), np.ones((4, 58, 77), np.float32), np.ones((20, 77), np.float32)
    y = oracle.gmm(x, A, gs)
    assert np.all(y[:17] == 58) and not np.any(y[17:])
    dA = oracle.tgmm(x, dy, gs)
    for gi, s in enumerate(gs):
        assert np.all(dA[gi] == s)


def test_trans_rhs_equals_plain_on_transposed_weights():
    """tests.py:156-161."""
    rng = np.random.default_rng(3)
    x = rng.normal(size=(40, 16)).astype(np.float32)
    A = rng.normal(size=(3, 16, 24)).astype(np.float32)
    gs = [10, 5, 20]
    np.testing.assert_array_equal(oracle.gmm(x, A, gs), oracle.gmm(x, np.swapaxes(A, 1, 2).copy(), gs, trans_rhs=True))


def test_brute_force_tiny():
    """Element-by-element triple loop on a tiny case: catches a transposed operand or an off-by-one group boundary."""
    rng = np.random.default_rng(4)
    m, k, n = 9, 3, 4
    gs = [2, 0, 4, 1]
    x, A, dy = rng.normal(size=(m, k)), rng.normal(size=(4, k, n)), rng.normal(size=(m, n))
    group_of_row = [0, 0, 2, 2, 2, 2, 3, None, None]
    y = np.zeros((m, n))
    dA = np.zeros((4, k, n))
    for r in range(m):
        gi = group_of_row[r]
        if gi is None:
            continue
        for j in range(n):
            for kk in range(k):
                y[r, j] += x[r, kk] * A[gi, kk, j]
                dA[gi, kk, j] += x[r, kk] * dy[r, j]
    np.testing.assert_allclose(oracle.gmm(x, A, gs, out_dtype="float32", acc=np.float64), y, rtol=1e-12, atol=1e-14)
    np.testing.assert_allclose(oracle.tgmm(x, dy, gs, out_dtype="float32", acc=np.float64), dA, rtol=1e-12, atol=1e-14)


# ---- VJP wiring (gpu_ragged_dot.py:383-402) ---------------------------------------------------------------------------

@pytest.mark.parametrize("trans_rhs", [False, True])
def test_vjp_adjoint_identities_and_finite_differences(trans_rhs):
    rng = np.random.default_rng(5)
    m, k, n, g = 30, 7, 5, 4
    gs = [8, 0, 15, 4]  # 27 of 30 rows used
    x = rng.normal(size=(m, k))
    A = rng.normal(size=(g, n, k) if trans_rhs else (g, k, n))
    dout = rng.normal(size=(m, n))
    f = lambda x_, A_: oracle.gmm(x_, A_, gs, trans_rhs=trans_rhs, out_dtype="float32", acc=np.float64)
    dx, dA, dgs = oracle.gmm_vjp(x, A, gs, dout, trans_rhs=trans_rhs, out_dtype="float32", acc=np.float64)
    assert dgs is None and dx.shape == x.shape and dA.shape == A.shape
    # <dout, f(x, A)> is bilinear: it equals <dx, x> and <dA, A>
    lhs = np.sum(dout * f(x, A))
    np.testing.assert_allclose(np.sum(dx * x), lhs, rtol=1e-10)
    np.testing.assert_allclose(np.sum(dA * A), lhs, rtol=1e-10)
    # central differences of s(x, A) = <dout, f(x, A)> along random directions
    vx, vA = rng.normal(size=x.shape), rng.normal(size=A.shape)
    eps = 1e-6
    num_x = (np.sum(dout * f(x + eps * vx, A)) - np.sum(dout * f(x - eps * vx, A))) / (2 * eps)
    num_A = (np.sum(dout * f(x, A + eps * vA)) - np.sum(dout * f(x, A - eps * vA))) / (2 * eps)
    np.testing.assert_allclose(np.sum(dx * vx), num_x, rtol=1e-6)
    np.testing.assert_allclose(np.sum(dA * vA), num_A, rtol=1e-6)
    assert not np.any(dx[27:]) and not np.any(dA[1])


def test_tgmm_vjp_adjoint_identities_and_finite_differences():
    """The VJP of tgmm (what gpu_ragged_dot.py:431-450 intends): s(x, y) = <dout, tgmm(x, y)> is bilinear, so
    <dx, x> = <dy, y> = s, and its directional derivatives are <dx, vx> and <dy, vy>.  A swapped operand, a missing
    transpose or cotangents leaking into rows past sum(group_sizes) fails one of these."""
    rng = np.random.default_rng(6)
    m, k, n, g = 30, 7, 5, 4
    gs = [8, 0, 15, 4]  # 27 of 30 rows used, one empty group
    x, y = rng.normal(size=(m, k)), rng.normal(size=(m, n))
    dout = rng.normal(size=(g, k, n))
    f = lambda x_, y_: oracle.tgmm(x_, y_, gs, out_dtype="float32", acc=np.float64)
    dx, dy, dgs = oracle.tgmm_vjp(x, y, gs, dout, out_dtype="float32", acc=np.float64)
    assert dgs is None and dx.shape == x.shape and dy.shape == y.shape
    s = np.sum(dout * f(x, y))
    np.testing.assert_allclose(np.sum(dx * x), s, rtol=1e-10)
    np.testing.assert_allclose(np.sum(dy * y), s, rtol=1e-10)
    vx, vy = rng.normal(size=x.shape), rng.normal(size=y.shape)
    eps = 1e-6
    num_x = (np.sum(dout * f(x + eps * vx, y)) - np.sum(dout * f(x - eps * vx, y))) / (2 * eps)
    num_y = (np.sum(dout * f(x, y + eps * vy)) - np.sum(dout * f(x, y - eps * vy))) / (2 * eps)
    np.testing.assert_allclose(np.sum(dx * vx), num_x, rtol=1e-6)
    np.testing.assert_allclose(np.sum(dy * vy), num_y, rtol=1e-6)
    assert not np.any(dx[27:]) and not np.any(dy[27:])
    # per group, by the definition: dx_g = y_g dout_g^T, dy_g = x_g dout_g
    np.testing.assert_allclose(dx[8:23], y[8:23] @ dout[2].T, rtol=1e-12)
    np.testing.assert_allclose(dy[23:27], x[23:27] @ dout[3], rtol=1e-12)


def test_group_offset_is_the_product_with_the_other_groups_weights_zero():
    """group_offset (A holds a slice of the groups) reduces to the pinned definition: the same product with zero
    weights for the groups outside the slice; tgmm's slices are rows [o, o + gl) of the full result; the VJP wiring
    satisfies the adjoint identities."""
    rng = np.random.default_rng(8)
    m, k, n, G = 40, 6, 5, 7
    gs = [5, 0, 9, 3, 8, 0, 10]  # 35 of 40 rows
    x, A, dy = rng.normal(size=(m, k)), rng.normal(size=(G, k, n)), rng.normal(size=(m, n))
    f64 = dict(out_dtype="float32", acc=np.float64)
    for o, gl in ((0, 7), (2, 3), (4, 3), (6, 1), (1, 1)):
        A0 = np.zeros_like(A)
        A0[o:o + gl] = A[o:o + gl]
        np.testing.assert_array_equal(oracle.gmm(x, A[o:o + gl], gs, group_offset=o, **f64), oracle.gmm(x, A0, gs, **f64))
        At = np.swapaxes(A, 1, 2).copy()
        np.testing.assert_array_equal(oracle.gmm(x, At[o:o + gl], gs, trans_rhs=True, group_offset=o, **f64), oracle.gmm(x, A0, gs, **f64))
        np.testing.assert_array_equal(oracle.tgmm(x, dy, gs, group_offset=o, num_actual_groups=gl, **f64), oracle.tgmm(x, dy, gs, **f64)[o:o + gl])
        dx, dA, _ = oracle.gmm_vjp(x, A[o:o + gl], gs, dy, group_offset=o, **f64)
        s = np.sum(dy * oracle.gmm(x, A[o:o + gl], gs, group_offset=o, **f64))
        np.testing.assert_allclose(np.sum(dx * x), s, rtol=1e-10)
        np.testing.assert_allclose(np.sum(dA * A[o:o + gl]), s, rtol=1e-10)
        assert dA.shape == (gl, k, n)


# ---- the loop-nest restatement against the definition, on the reference's own grid ----------------------------------

GRID = util.reference_grid(36, seed=1)


@pytest.mark.parametrize("c", GRID, ids=[util.case_id(c) for c in GRID])
def test_blocked_restatement_matches_definition(c):
    lhs, rhs, dout, gs, target_m = util.make_case(c["seed"], c["m"], c["k"], c["n"], c["g"], c["fill_in"], c["random_inputs"])
    kw = dict(block_m=c["block_m"], block_k=c["block_k"], block_n=c["block_n"])
    y = oracle.gmm_blocked(lhs, rhs, gs, chunk_m=c["chunk_m"], **kw)
    y_ref = oracle.gmm(lhs, rhs, gs)
    if target_m > 0:
        assert not np.isnan(y).any(), "the reference's programs write every element when some group is non-empty"
        util.assert_close_rows(y, y_ref, target_m, util.BF16_EPS, "gmm_blocked")
        assert not np.any(y[target_m:])
    yt = oracle.gmm_blocked(lhs, np.ascontiguousarray(np.swapaxes(rhs, 1, 2)), gs, trans_rhs=True, chunk_m=c["chunk_m"], **kw)
    if target_m > 0:
        util.assert_close_rows(yt, y_ref, target_m, util.BF16_EPS, "gmm_blocked trans_rhs")
    dA = oracle.tgmm_blocked(lhs, dout, gs, **kw)
    assert not np.isnan(dA).any()
    util.assert_close_groups(dA, oracle.tgmm(lhs, dout, gs), gs != 0, util.TGMM_BF16_EPS, "tgmm_blocked")
    assert not np.any(dA[gs == 0])
    if not c["random_inputs"]:
        assert np.all(y[:target_m] == c["k"])


def test_blocked_all_empty_groups_leaves_output_untouched():
    """gpu_ragged_dot.py:157: with every group empty no program is 'last', so the reference never writes y.  The HIP
    path deliberately differs (it zero-fills); this records what the reference itself defines."""
    y = oracle.gmm_blocked(np.ones((16, 16), np.float32), np.ones((2, 16, 16), np.float32), [0, 0], fill=np.nan)
    assert np.isnan(y).all()


# ---- metric and generators -------------------------------------------------------------------------------------------

def test_err_fn_known_values():
    a = np.array([[3.0, 4.0], [0.0, 0.0]])
    b = np.array([[0.0, 0.0], [0.0, 0.0]])
    e = oracle.err_fn(a, b)
    assert e[0] == pytest.approx(5.0 / 1e-7) and e[1] == 0.0
    assert oracle.err_fn(a, b, mask=np.array([False, True])).tolist() == [0.0, 0.0]
    assert oracle.err_fn(np.array([[1.0, 1.0]]), np.array([[1.0, 0.0]]))[0] == pytest.approx(1.0)


def test_generate_group_sizes_sums():
    for seed in range(10):
        for g, t in ((8, 128), (16, 120), (16, 0), (8, 86)):
            gs = oracle.generate_group_sizes(seed, g, t)
            assert gs.dtype == np.int32 and gs.sum() == t and np.all(gs >= 0) and gs.size == g


# ---------------------------------------------------------------------------------------------------------------------
# float8 e4m3fn on the host
# ---------------------------------------------------------------------------------------------------------------------

def test_float8_decode_known_values_and_torch():
    """Values fixed by the E4M3 definition (bias 7, subnormals mantissa x 2^-9, max 448, S.1111.111 NaN, no infinities),
    then all 256 codes against torch's own CPU conversion - an independent implementation."""
    torch = pytest.importorskip("torch")
    dec = oracle.float8_e4m3fn_to_f32
    known = {0x00: 0.0, 0x01: 2.0 ** -9, 0x07: 7 * 2.0 ** -9, 0x08: 2.0 ** -6, 0x0F: 1.875 * 2.0 ** -6, 0x38: 1.0, 0x3C: 1.5,
             0x40: 2.0, 0x77: 1.875 * 2.0 ** 7, 0x78: 256.0, 0x7E: 448.0, 0xB8: -1.0, 0xFE: -448.0, 0x81: -(2.0 ** -9)}
    for code, val in known.items():
        assert float(dec(np.array([code], np.uint8))[0]) == val, hex(code)
    assert np.signbit(dec(np.array([0x80], np.uint8))[0]) and dec(np.array([0x80], np.uint8))[0] == 0.0
    assert np.isnan(dec(np.array([0x7F, 0xFF], np.uint8))).all()
    codes = np.arange(256, dtype=np.uint8)
    mine = dec(codes)
    assert np.isfinite(mine).sum() == 254 and np.all(np.diff(mine[:127]) > 0)
    theirs = torch.from_numpy(codes).view(torch.float8_e4m3fn).to(torch.float32).numpy()
    assert np.array_equal(np.isnan(mine), np.isnan(theirs))
    assert np.array_equal(mine[np.isfinite(mine)], theirs[np.isfinite(theirs)])
    # every e4m3 value is a bf16 value: the kernels' widening is exact
    assert np.array_equal(oracle.round_to(mine[np.isfinite(mine)], "bfloat16"), mine[np.isfinite(mine)])


def test_float8_encode_round_trip_ties_and_saturation():
    torch = pytest.importorskip("torch")
    enc, dec = oracle.f32_to_float8_e4m3fn, oracle.float8_e4m3fn_to_f32
    codes = np.arange(256, dtype=np.uint8)
    finite = codes[(codes & 0x7F) != 0x7F]
    assert np.array_equal(enc(dec(finite)), finite)
    assert enc(np.array([1.0625]))[0] == 0x38 and enc(np.array([1.1875]))[0] == 0x3A  # ties go to the even code
    assert enc(np.array([1e9]))[0] == 0x7E and enc(np.array([-1e9]))[0] == 0xFE and enc(np.array([np.nan]))[0] == 0x7F
    x = (np.random.default_rng(0).normal(size=50000) * 4).astype(np.float32)
    assert np.array_equal(enc(x), torch.from_numpy(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy())
