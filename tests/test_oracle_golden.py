"""CPU tests: the oracle against the reference-held vectors, closed forms and brute force.

These pin the CPU restatement (oracle/nd4j_oracle.c) before any GPU result is compared with it.
"""
import math

import numpy as np
import pytest

from conftest import assert_close, materialize


# ---- hash: libnd4j/tests_cpu/layers_tests/HashUtilsTests.cpp:28-41 -------------------------------------------
def test_hash_reference_vectors(oracle):
    assert oracle.hash_name("Conv2D") == -1637140380760460323
    assert oracle.hash_name("switch") == -1988317239813741487


# ---- shape walk: brute force against numpy strided views -------------------------------------------------
@pytest.mark.parametrize("shape,perm", [((5,), (0,)), ((3, 4), (1, 0)), ((2, 3, 4), (2, 0, 1)), ((2, 3, 4, 5), (0, 2, 1, 3)),
                                        ((2, 2, 3, 2, 2), (4, 3, 2, 1, 0)), ((2, 1, 3, 1, 2, 2), (5, 0, 3, 2, 1, 4))])
def test_offset_walk_matches_numpy(oracle, shape, perm):
    base = np.arange(int(np.prod(shape)), dtype=np.float32).reshape(shape)
    view = base.transpose(perm)
    si = oracle.shape_info(view)
    flat = base.ravel()
    logical = view.ravel()  # row-major over the VIEW's shape
    for i in range(view.size):
        assert flat[oracle.offset(si, i)] == logical[i]


def test_offset_walk_f_order_is_row_major_over_shape(oracle):
    a = np.asfortranarray(np.arange(12, dtype=np.float32).reshape(3, 4))
    si = oracle.shape_info(a)
    assert chr(int(si[-1])) == "f"
    buf = a.ravel(order="K")
    assert [buf[oracle.offset(si, i)] for i in range(12)] == list(range(12))


@pytest.mark.parametrize("shape,dims", [((5, 5), [1]), ((5, 5), [0]), ((2, 3, 4), [1, 2]), ((2, 3, 4), [0, 2]), ((2, 3, 4, 5), [1]),
                                        ((3, 4), [0, 1])])
def test_tad_matches_numpy(oracle, shape, dims):
    a = np.arange(int(np.prod(shape)), dtype=np.float32).reshape(shape)
    tsi, offs = oracle.tad(a, dims)
    if len(dims) == a.ndim:
        assert list(offs) == list(range(a.size))
        return
    other = [d for d in range(a.ndim) if d not in dims]
    moved = np.moveaxis(a, other, list(range(len(other))))
    firsts = moved.reshape((-1,) + tuple(a.shape[d] for d in dims))[(slice(None),) + (0,) * len(dims)]
    assert list(offs) == [int(v) for v in firsts]
    rank = int(tsi[0])
    assert list(tsi[1:1 + rank]) == [a.shape[d] for d in dims]
    assert list(tsi[1 + rank:1 + 2 * rank]) == [a.strides[d] // 4 for d in dims]


# ---- half conversions ------------------------------------------------------------------------------------
def test_f16_conversion_matches_numpy(oracle):
    rng = np.random.default_rng(7)
    vals = np.concatenate([rng.normal(0, 1, 2000), rng.normal(0, 1e-6, 500), rng.normal(0, 3e4, 500),
                           [0.0, -0.0, np.inf, -np.inf, 65504.0, 65520.0, 6e-8, 5.96e-8, 2.98e-8, 1e-9]]).astype(np.float32)
    L = oracle.lib()
    got = np.array([L.orc_f32_to_f16(float(v)) for v in vals], dtype=np.uint16)
    want = vals.astype(np.float16).view(np.uint16)
    assert (got == want).all()
    back = np.array([L.orc_f16_to_f32(int(h)) for h in range(0, 65536, 7)], dtype=np.float32)
    ref = np.arange(0, 65536, 7, dtype=np.uint16).view(np.float16).astype(np.float32)
    assert np.array_equal(back, ref, equal_nan=True)


def test_bf16_rounding_is_nearest_even(oracle):
    L = oracle.lib()
    one = np.float32(1.0).view(np.uint32)
    for bits, want in [(one + 0x8000, 0x3F80), (one + 0x8001, 0x3F81), (one + 0x18000, 0x3F82), (one + 0x7FFF, 0x3F80)]:
        assert L.orc_f32_to_bf16(float(np.uint32(bits).view(np.float32))) == want
    assert L.orc_f32_to_bf16(float("nan")) == 0x7FC0
    assert (oracle.f32_to_bf16(np.array([1.0, np.nan], np.float32)) == np.array([0x3F80, 0x7FC0], np.uint16)).all()


# ---- pairwise: NativeOpsTests.cpp:170-186 (5x5 linspace + 2 -> element 5 == 8), bit-exact vs numpy ---------
def test_pairwise_reference_vector(oracle):
    x = np.linspace(1, 25, 25, dtype=np.float32).reshape(5, 5)
    y = np.full((5, 5), 2, dtype=np.float32)
    z = oracle.pairwise(0, x, y, np.zeros_like(x))
    assert z.ravel()[5] == 8


@pytest.mark.parametrize("op,fn", [(0, np.add), (2, np.divide), (3, np.multiply), (6, np.subtract), (7, np.maximum), (8, np.minimum),
                                   (5, lambda a, b: b - a), (11, lambda a, b: b / a), (1, lambda a, b: b), (20, lambda a, b: (a - b) * (a - b))])
def test_pairwise_bit_exact_vs_numpy(oracle, op, fn):
    rng = np.random.default_rng(op)
    x = rng.uniform(-1, 1, (37, 19)).astype(np.float32)
    y = rng.uniform(0.5, 1.5, (37, 19)).astype(np.float32)
    z = oracle.pairwise(op, x, y.T.copy().T, np.zeros_like(x))
    assert np.array_equal(z, fn(x, y).astype(np.float32))


def test_pairwise_strided_operands(oracle):
    rng = np.random.default_rng(3)
    x = rng.uniform(-1, 1, (6, 8)).astype(np.float32)
    y = rng.uniform(-1, 1, (8, 6)).astype(np.float32)
    z = oracle.pairwise(0, x, y.T, np.zeros((6, 8), np.float32))
    assert np.array_equal(z, x + y.T)


def test_pairwise_rejects_foreign_output_type(oracle):
    x = np.zeros(4, np.float32)
    with pytest.raises(ValueError):
        oracle.pairwise(0, x, x, np.zeros(4, np.float64))


# ---- transforms: NativeOpsTests.cpp:658-760, TestTransformOpValidation.java:1043-1054 -----------------------
def test_transform_float_sqrt_exact(oracle):
    x = np.linspace(1, 25, 25, dtype=np.float32).reshape(5, 5)
    assert np.array_equal(oracle.transform_float(1, x, np.zeros_like(x)), np.sqrt(x))
    assert np.array_equal(oracle.transform_float(3, x, np.zeros_like(x)), (np.float32(1) / np.sqrt(x)).astype(np.float32))


def test_tanh_formula_against_fp64(oracle):
    x = np.linspace(-2, 2, 4001, dtype=np.float32)
    z = oracle.transform_strict(29, x, np.zeros_like(x))
    assert np.abs(z.astype(np.float64) - np.tanh(x.astype(np.float64))).max() <= 2e-7
    assert (np.sign(z) == np.sign(x)).all()
    big = np.array([-50, 50, -1e4, 1e4], np.float32)
    assert np.array_equal(oracle.transform_strict(29, big, np.zeros_like(big)), np.array([-1, 1, -1, 1], np.float32))


def test_gelu_closed_forms(oracle):
    # GELU = x * sigmoid(1.702 x); PreciseGELU = x/2 (1 + tanh(sqrt(2/pi) (x + (0.044715 x)^3))) -- the cube wraps 0.044715*x
    x = np.linspace(-4, 4, 801, dtype=np.float32)
    x64 = x.astype(np.float64)
    g = oracle.transform_strict(53, x, np.zeros_like(x))
    assert_close(g, x64 / (1 + np.exp(-1.702 * x64)), 1e-5, 1e-6, "gelu")
    pg = oracle.transform_strict(55, x, np.zeros_like(x))
    assert_close(pg, 0.5 * x64 * (1 + np.tanh(math.sqrt(2 / math.pi) * (x64 + (0.044715 * x64) ** 3))), 1e-5, 1e-6, "precise gelu")
    # the textbook form with 0.044715*x^3 differs measurably: make sure we did not implement that one
    textbook = 0.5 * x64 * (1 + np.tanh(math.sqrt(2 / math.pi) * (x64 + 0.044715 * x64 ** 3)))
    assert np.abs(pg - textbook).max() > 1e-2


def test_sigmoid_exp_log(oracle):
    x = np.linspace(-6, 6, 1201, dtype=np.float32)
    assert_close(oracle.transform_strict(26, x, np.zeros_like(x)), 1 / (1 + np.exp(-x.astype(np.float64))), 1e-6, 1e-7, "sigmoid")
    assert_close(oracle.transform_strict(23, x, np.zeros_like(x)), np.exp(x.astype(np.float64)), 2e-7, 0, "exp")
    p = np.abs(x) + 0.5
    assert_close(oracle.transform_strict(24, p, np.zeros_like(p)), np.log(p.astype(np.float64)), 2e-7, 1e-7, "log")


# ---- reductions: NativeOpsTests.cpp:209-238 (Mean of 1..25 = 13, Sum = 325), LegacyOpsTests.cpp:151-277 --------
def test_reduce_reference_vectors(oracle):
    x = np.linspace(1, 25, 25, dtype=np.float32).reshape(5, 5)
    assert oracle.reduce_float(0, x, np.zeros((), np.float32)) == 13
    assert oracle.reduce_same(0, x, np.zeros((), np.float32)) == 325
    assert list(oracle.reduce_same(0, x, np.zeros(5, np.float32), [1])) == [15, 40, 65, 90, 115]
    assert list(oracle.reduce_same(1, x, np.zeros(5, np.float32), [0])) == [21, 22, 23, 24, 25]
    assert list(oracle.reduce_float(0, x, np.zeros(5, np.float32), [-1])) == [3, 8, 13, 18, 23]


def test_reduce_sum_is_sequential_fp32(oracle):
    rng = np.random.default_rng(11)
    x = rng.uniform(-1, 1, (7, 1000)).astype(np.float32)
    z = oracle.reduce_same(0, x, np.zeros(7, np.float32), [1])
    for r in range(7):
        s = np.float32(0)
        for v in x[r]:
            s = np.float32(v + s)
        assert z[r] == s


@pytest.mark.parametrize("op,fn", [(1, lambda a, ax: a.max(ax)), (2, lambda a, ax: a.min(ax)), (4, lambda a, ax: np.abs(a).sum(ax)),
                                   (5, lambda a, ax: np.abs(a).max(ax)), (6, lambda a, ax: np.abs(a).min(ax)), (3, lambda a, ax: a.prod(ax))])
def test_reduce_same_ops(oracle, op, fn):
    rng = np.random.default_rng(op)
    x = rng.uniform(0.5, 1.5, (4, 6, 5)).astype(np.float32) * rng.choice([-1, 1], (4, 6, 5)).astype(np.float32)
    z = oracle.reduce_same(op, x, np.zeros((4, 5), np.float32), [1])
    assert_close(z, fn(x.astype(np.float64), 1), 1e-5, 1e-6, "reduce_same %d" % op)


@pytest.mark.parametrize("op,fn", [(0, lambda a, ax: a.mean(ax)), (1, lambda a, ax: np.abs(a).mean(ax)), (2, lambda a, ax: np.abs(a).sum(ax)),
                                   (3, lambda a, ax: np.sqrt((a * a).sum(ax))), (4, lambda a, ax: np.abs(a).max(ax)), (7, lambda a, ax: (a * a).sum(ax))])
def test_reduce_float_ops(oracle, op, fn):
    rng = np.random.default_rng(op)
    x = rng.normal(0, 1, (3, 4, 50)).astype(np.float32)
    z = oracle.reduce_float(op, x, np.zeros((3, 50), np.float32), [1])
    assert_close(z, fn(x.astype(np.float64), 1), 1e-5, 1e-6, "reduce_float %d" % op)
    z2 = oracle.reduce_float(op, x.transpose(2, 0, 1), np.zeros((50, 3), np.float32), [2])
    assert_close(z2, fn(x.astype(np.float64), 1).T, 1e-5, 1e-6, "reduce_float strided %d" % op)


# ---- index reduce: NativeOpsTests.cpp:84-117 (-> 4, -> 24), LegacyOpsTests.cpp:279-310 (dim 1 -> all 4) -------
def test_index_reduce_reference_vectors(oracle):
    x = np.linspace(1, 5, 5, dtype=np.float32)
    assert oracle.index_reduce(0, x, np.zeros((), np.int64)) == 4
    x = np.linspace(1, 25, 25, dtype=np.float32).reshape(5, 5)
    assert oracle.index_reduce(0, x, np.zeros((), np.int64)) == 24
    assert list(oracle.index_reduce(0, x, np.zeros(5, np.int64), [1])) == [4] * 5
    assert list(oracle.index_reduce(1, x, np.zeros(5, np.int64), [1])) == [0] * 5


def test_index_reduce_ties_nan_inf(oracle):
    inf, nan = np.inf, np.nan
    rows = np.array([[1, 3, 3, 2], [nan, 1, 2, 2], [-inf, -inf, -inf, -inf], [nan, nan, nan, nan], [nan, -inf, 5, nan], [2, 2, 2, 2]], np.float32)
    assert list(oracle.index_reduce(0, rows, np.zeros(6, np.int64), [1])) == [1, 2, 0, 0, 2, 0]
    assert list(oracle.index_reduce(1, rows, np.zeros(6, np.int64), [1])) == [0, 1, 0, 0, 1, 0]
    rows2 = np.array([[1, -3, 3, 2], [0, 0, 0, 0], [nan, -1, 1, 0]], np.float32)
    assert list(oracle.index_reduce(2, rows2, np.zeros(3, np.int64), [1])) == [1, 0, 1]
    assert list(oracle.index_reduce(3, rows2, np.zeros(3, np.int64), [1])) == [0, 0, 3]


def test_index_reduce_brute_force(oracle):
    rng = np.random.default_rng(5)
    x = rng.integers(-3, 4, (6, 7, 8)).astype(np.float32)   # many ties
    for dims in ([2], [1], [0], [1, 2], [0, 2]):
        out_shape = [s for i, s in enumerate(x.shape) if i not in dims]
        z = oracle.index_reduce(0, x, np.zeros(out_shape, np.int64), dims)
        other = [d for d in range(3) if d not in dims]
        moved = np.transpose(x, other + dims).reshape(int(np.prod(out_shape)), -1)
        assert list(z.ravel()) == [int(np.argmax(r)) for r in moved]     # numpy argmax returns the first maximum


# ---- golden vectors held by the reference's own unit tests ------------------------------------------------------
def _cases(golden, op):
    return [c for c in golden if c["op"] == op]


def test_golden_matmul(oracle, golden):
    cases = _cases(golden, "matmul")
    assert len(cases) >= 35
    for c in cases:
        x, y = (materialize(s) for s in c["inputs"])
        exp = materialize(c["expected"])
        z = materialize(c["initial_output"]).copy(order="K") if "initial_output" in c else np.zeros_like(exp)
        ia = c["iargs"] + [0] * (3 - len(c["iargs"]))
        alpha = c["targs"][0] if len(c["targs"]) > 0 else 1.0
        beta = c["targs"][1] if len(c["targs"]) > 1 else 0.0
        oracle.matmul(x, y, z, bool(ia[0]), bool(ia[1]), bool(ia[2]), alpha, beta, accumulate=2)
        assert_close(z, exp, 1e-6, 1e-9, c["name"])


def test_golden_softmax(oracle, golden):
    cases = _cases(golden, "softmax")
    assert len(cases) == 12
    for c in cases:
        x = materialize(c["inputs"][0])
        exp = materialize(c["expected"])
        dim = c["iargs"][0] if c["iargs"] else -1
        z = np.zeros_like(x)
        oracle.softmax(x, z, dim)
        # the reference prints its expectations with 5-6 significant digits (equalsTo uses eps 1e-5)
        assert_close(z, exp, 1e-4, 1e-5, c["name"])


def test_golden_argmax(oracle, golden):
    cases = _cases(golden, "argmax")
    assert len(cases) >= 4
    for c in cases:
        x = materialize(c["inputs"][0])
        dims = c["iargs"] if len(c["inputs"]) == 1 else [int(v) for v in materialize(c["inputs"][1]).ravel()]
        exp = materialize(c["expected"])
        z = np.zeros(exp.shape, np.int64)
        oracle.index_reduce(0, x, z, dims)
        assert np.array_equal(z, exp.astype(np.int64)), c["name"]


# ---- matmul / softmax / layer_norm against mathematics -----------------------------------------------------------
def test_matmul_transposes_and_batches(oracle):
    rng = np.random.default_rng(2)
    a = rng.normal(0, 1, (3, 5, 7)).astype(np.float32)
    b = rng.normal(0, 1, (3, 7, 4)).astype(np.float32)
    want = a.astype(np.float64) @ b.astype(np.float64)
    assert_close(oracle.matmul(a, b, np.zeros((3, 5, 4), np.float32)), want, 1e-5, 1e-5, "plain")
    assert_close(oracle.matmul(a.transpose(0, 2, 1).copy(), b, np.zeros((3, 5, 4), np.float32), trans_x=True), want, 1e-5, 1e-5, "transX")
    assert_close(oracle.matmul(a, b.transpose(0, 2, 1).copy(), np.zeros((3, 5, 4), np.float32), trans_y=True), want, 1e-5, 1e-5, "transY")
    zt = oracle.matmul(b.transpose(0, 2, 1).copy(), a.transpose(0, 2, 1).copy(), np.zeros((3, 5, 4), np.float32), trans_z=True)
    # transZ swaps the operands and flips the flags: z = (b^T)^T' ... = a @ b for these operands
    assert_close(zt, want, 1e-5, 1e-5, "transZ")
    c0 = rng.normal(0, 1, (3, 5, 4)).astype(np.float32)
    z = c0.copy()
    oracle.matmul(a, b, z, alpha=0.5, beta=2.0)
    assert_close(z, 0.5 * want + 2.0 * c0, 1e-5, 1e-5, "alpha/beta")


def test_matmul_literal_half_accumulation_is_worse(oracle):
    # usualGemm accumulates in the output type: for bf16 and K = 1024 it drifts far from the fp32-accumulated value
    rng = np.random.default_rng(4)
    K = 1024
    a = oracle.Arr(oracle.f32_to_bf16(rng.normal(0, 1 / math.sqrt(K), (4, K)).astype(np.float32)), oracle.BFLOAT16)
    b = oracle.Arr(oracle.f32_to_bf16(rng.normal(0, 1 / math.sqrt(K), (K, 4)).astype(np.float32)), oracle.BFLOAT16)
    z0 = oracle.Arr(np.zeros((4, 4), np.uint16), oracle.BFLOAT16)
    z1 = oracle.Arr(np.zeros((4, 4), np.uint16), oracle.BFLOAT16)
    oracle.matmul(a, b, z0, accumulate=0)
    oracle.matmul(a, b, z1, accumulate=1)
    exact = oracle.bf16_to_f32(a.a).astype(np.float64) @ oracle.bf16_to_f32(b.a).astype(np.float64)
    e0 = np.abs(oracle.bf16_to_f32(z0.a) - exact).max()
    e1 = np.abs(oracle.bf16_to_f32(z1.a) - exact).max()
    assert e1 <= 2 ** -8 * np.abs(exact).max() + 1e-6
    assert e0 >= e1


def test_softmax_vs_numpy_and_edges(oracle):
    rng = np.random.default_rng(6)
    x = rng.normal(0, 2, (4, 3, 33)).astype(np.float32)
    x64 = x.astype(np.float64)
    for dim in (0, 1, 2):
        e = np.exp(x64 - x64.max(dim, keepdims=True))
        assert_close(oracle.softmax(x, np.zeros_like(x), dim), e / e.sum(dim, keepdims=True), 1e-5, 1e-7, "softmax dim %d" % dim)
    # strided input, dense output: fallback branch, same numbers for finite data
    xt = np.ascontiguousarray(x.transpose(0, 2, 1))
    e = np.exp(x64 - x64.max(2, keepdims=True))
    assert_close(oracle.softmax(xt.transpose(0, 2, 1), np.zeros_like(x), 2), e / e.sum(2, keepdims=True), 1e-5, 1e-7, "softmax strided")
    # clamp semantics of the same-shape branch (source only): inf counts as max + 88, so it takes all the mass
    row = np.array([[0.0, np.inf, 1.0, -np.inf]], np.float32)
    z = oracle.softmax(row.repeat(2, 0), np.zeros((2, 4), np.float32), 1)
    assert z[0, 1] == pytest.approx(1.0) and z[0, 0] < 1e-30 and z[0, 3] < 1e-30
    # a row of equal values is uniform; shifting a row does not change the result
    assert_close(oracle.softmax(np.full((2, 8), 3.0, np.float32), np.zeros((2, 8), np.float32)), np.full((2, 8), 0.125), 1e-6, 0, "uniform")
    assert_close(oracle.softmax(x + 5, np.zeros_like(x)), oracle.softmax(x, np.zeros_like(x)), 2e-5, 1e-7, "shift invariance")


def test_layer_norm_closed_form(oracle):
    rng = np.random.default_rng(8)
    x = rng.normal(0.3, 1.7, (4, 6, 40)).astype(np.float32)
    g = rng.normal(1, 0.02, 40).astype(np.float32)
    b = rng.normal(0, 0.02, 40).astype(np.float32)
    x64 = x.astype(np.float64)
    want = (x64 - x64.mean(2, keepdims=True)) / np.sqrt(x64.var(2, keepdims=True) + 1e-5) * g + b
    assert_close(oracle.layer_norm(x, g, b, np.zeros_like(x), [2], channels_first=False), want, 1e-5, 1e-5, "NHWC last axis")
    assert_close(oracle.layer_norm(x, g, None, np.zeros_like(x), [2], channels_first=False), want - b, 1e-5, 1e-5, "no bias")
    # channels first (gain along dim 1), statistics over dims 1..3 of a 4-D array (TestLayerOpValidation.java:1188-1333)
    x4 = rng.normal(0, 1, (3, 5, 4, 2)).astype(np.float32)
    g4 = rng.normal(1, 0.1, 5).astype(np.float32)
    b4 = rng.normal(0, 0.1, 5).astype(np.float32)
    x464 = x4.astype(np.float64)
    want4 = (x464 - x464.mean((1, 2, 3), keepdims=True)) / np.sqrt(x464.var((1, 2, 3), keepdims=True) + 1e-5) * g4[None, :, None, None] + b4[None, :, None, None]
    assert_close(oracle.layer_norm(x4, g4, b4, np.zeros_like(x4), [1, 2, 3], channels_first=True), want4, 1e-5, 1e-5, "NCHW")
    # a constant row has zero variance: output = bias (eps keeps the division finite)
    xc = np.full((2, 40), 7.0, np.float32)
    assert_close(oracle.layer_norm(xc, g, b, np.zeros_like(xc), [1], channels_first=False), np.tile(b, (2, 1)), 0, 1e-6, "constant row")


def test_attention_is_matmul_softmax_matmul(oracle):
    rng = np.random.default_rng(9)
    B, T, D = 2, 9, 8
    q, k, v = (rng.normal(0, 1, (B, T, D)).astype(np.float32) for _ in range(3))
    out = np.zeros((B, T, D), np.float32)
    w = np.zeros((B, T, T), np.float32)
    lg = np.zeros((B, T, T), np.float32)
    oracle.attention_v2(q, v, k, out, w, lg, scale=0.5, causal=False)
    s = 0.5 * (q.astype(np.float64) @ k.astype(np.float64).transpose(0, 2, 1))
    e = np.exp(s - s.max(-1, keepdims=True))
    p = e / e.sum(-1, keepdims=True)
    assert_close(lg, s, 1e-5, 1e-6, "logits")
    assert_close(w, p, 1e-5, 1e-7, "weights")
    assert_close(out, p @ v.astype(np.float64), 1e-5, 1e-6, "out")
    oracle.attention_v2(q, v, k, out, w, lg, scale=0.5, causal=True)
    sm = np.where(np.tril(np.ones((T, T), bool)), s, -np.inf)
    e = np.exp(sm - sm.max(-1, keepdims=True))
    p = e / e.sum(-1, keepdims=True)
    assert_close(w, p, 1e-5, 1e-7, "causal weights")
    assert_close(out, p @ v.astype(np.float64), 1e-5, 1e-6, "causal out")
    assert (w[:, 0, 1:] < 1e-30).all() and w[:, 0, 0] == pytest.approx(1.0)


# ---- top_k --------------------------------------------------------------------------------------------------------------
def _topk_cases():
    import json
    import os
    with open(os.path.join(os.path.dirname(__file__), "golden", "top_k_vectors.json")) as f:
        return json.load(f)["cases"]


@pytest.mark.parametrize("case", _topk_cases(), ids=lambda c: c["name"])
def test_golden_top_k(oracle, case):
    """Known answers of the reference's own top_k tests ('f'-ordered buffers are laid out as the reference lays them out)."""
    order = case["order"].upper()
    x = np.array(case["x"], np.float64).reshape(case["shape"], order=order)
    v = np.zeros(case["zshape"], np.float64, order=order)
    i = np.zeros(case["zshape"], np.int64, order=order)
    oracle.top_k(x, v, i, case["k"], case["sort"])
    assert np.array_equal(v, np.array(case["v"], np.float64).reshape(case["zshape"], order=order))
    assert np.array_equal(i, np.array(case["i"], np.int64).reshape(case["zshape"], order=order))


def test_top_k_brute_force_on_distinct_values(oracle):
    rng = np.random.default_rng(7)
    for shape, k in [((5, 17), 3), ((2, 3, 40), 7), ((1, 1000), 40), ((4, 9), 9)]:
        x = rng.permutation(int(np.prod(shape))).astype(np.float32).reshape(shape)   # pairwise distinct
        v = np.zeros(shape[:-1] + (k,), np.float32)
        i = np.zeros(shape[:-1] + (k,), np.int64)
        oracle.top_k(x, v, i, k, True)
        want_i = np.argsort(-x, axis=-1, kind="stable")[..., :k]
        assert np.array_equal(i, want_i)
        assert np.array_equal(v, np.take_along_axis(x, want_i, -1))
        oracle.top_k(x, v, i, k, False)
        assert np.array_equal(i, np.sort(want_i, axis=-1))
