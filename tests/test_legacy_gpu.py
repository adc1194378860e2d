"""GPU parity tests of the legacy loops: every result comes out of libnd4jhip.so through the C ABI and is
compared with the CPU oracle on the same seeded inputs.

Gates (north star): index reductions bit-exact; fp32 elementwise / reduce |a-b| <= 1e-6 + 1e-5 |b|
(reductions: atol scaled by eps * sum|x|, the bound of a re-ordered fp32 sum); fp16/bf16 <= 1e-2.
"""
import numpy as np
import pytest

from conftest import assert_close
from deeplearning4j_amd.executioner import (IndexReduce, Pairwise, ReduceFloat, ReduceSame, Scalar, TransformFloat, TransformSame,
                                            TransformStrict)
from deeplearning4j_amd.ndarray import BFLOAT16, DOUBLE, FLOAT32, HALF, INT32, INT64, NDArray, bf16_bits_to_f32, f32_to_bf16_bits

pytestmark = pytest.mark.gpu

EPS32 = float(np.finfo(np.float32).eps)


def _oracle_arr(oracle, a, dtype):
    """numpy input -> (oracle operand, device array) in the requested storage type."""
    if dtype == BFLOAT16:
        bits = f32_to_bf16_bits(a)
        return oracle.Arr(bits, oracle.BFLOAT16), NDArray.from_numpy(bits, BFLOAT16)
    if dtype == HALF:
        h = a.astype(np.float16)
        return oracle.Arr(h), NDArray.from_numpy(h)
    if dtype == DOUBLE:
        d = a.astype(np.float64)
        return oracle.Arr(d), NDArray.from_numpy(d)
    f = a.astype(np.float32)
    return oracle.Arr(f), NDArray.from_numpy(f)


def _zeros_like(oracle, oa):
    return oracle.Arr(np.zeros(oa.a.shape, oa.a.dtype), oa.dt)


def _f(oa):
    return bf16_bits_to_f32(oa.a) if oa.dt == 17 else oa.a.astype(np.float64)


TOL = {FLOAT32: (1e-5, 1e-6), DOUBLE: (1e-12, 1e-13), HALF: (1e-2, 1e-3), BFLOAT16: (1e-2, 1e-3)}


# ---- pairwise ---------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("op", [Pairwise.Add, Pairwise.Subtract, Pairwise.Multiply, Pairwise.Divide, Pairwise.ReverseSubtract,
                                Pairwise.ReverseDivide, Pairwise.MaxPairwise, Pairwise.MinPairwise, Pairwise.CopyPws, Pairwise.SquaredSubtract])
def test_pairwise_fp32_bit_exact(ex, oracle, op):
    rng = np.random.default_rng(100 + op)
    x = rng.uniform(-1, 1, (257, 131)).astype(np.float32)
    y = (rng.uniform(0.5, 1.5, (257, 131)) * rng.choice([-1, 1], (257, 131))).astype(np.float32)
    want = oracle.pairwise(op, x, y, np.zeros_like(x))
    got = ex.exec_pairwise(op, NDArray.from_numpy(x), NDArray.from_numpy(y)).to_numpy()
    assert np.array_equal(got, want)          # one IEEE operation per element: identical bits


@pytest.mark.parametrize("dtype", [HALF, BFLOAT16, DOUBLE])
def test_pairwise_other_types(ex, oracle, dtype):
    rng = np.random.default_rng(7)
    a = rng.uniform(-2, 2, (64, 96))
    b = rng.uniform(0.5, 2, (64, 96))
    ox, dx = _oracle_arr(oracle, a, dtype)
    oy, dy = _oracle_arr(oracle, b, dtype)
    for op in (Pairwise.Add, Pairwise.Multiply, Pairwise.Divide):
        oz = _zeros_like(oracle, ox)
        oracle.pairwise(op, ox, oy, oz)
        got = ex.exec_pairwise(op, dx, dy).to_numpy()
        assert np.array_equal(got, oz.a), "single rounded operation must match bit for bit"


def test_pairwise_views_apply_offset_once(ex, oracle):
    # strided / permuted / offset operands: every operand walks its own descriptor, offset applied exactly once
    rng = np.random.default_rng(8)
    base_x = rng.uniform(-1, 1, (12, 40)).astype(np.float32)
    base_y = rng.uniform(-1, 1, (40, 12)).astype(np.float32)
    X = NDArray.from_numpy(base_x)
    Y = NDArray.from_numpy(base_y)
    xv = X.slice(0, 2, 10).slice(1, 5, 37)                  # [8, 32] view with an offset
    yv = Y.permute(1, 0).slice(0, 2, 10).slice(1, 5, 37)    # permuted + offset
    z = NDArray.empty((8, 32), FLOAT32)
    ex.exec_pairwise(Pairwise.Add, xv, yv, z)
    assert np.array_equal(z.to_numpy(), base_x[2:10, 5:37] + base_y.T[2:10, 5:37])
    # output into a view of a larger buffer leaves the rest untouched
    Zbig = NDArray.from_numpy(np.full((12, 40), -7, np.float32))
    ex.exec_pairwise(Pairwise.Multiply, xv, yv, Zbig.slice(0, 2, 10).slice(1, 5, 37))
    full = Zbig.to_numpy()
    assert np.array_equal(full[2:10, 5:37], base_x[2:10, 5:37] * base_y.T[2:10, 5:37])
    mask = np.ones((12, 40), bool)
    mask[2:10, 5:37] = False
    assert (full[mask] == -7).all()


def test_pairwise_f_order_and_rank5(ex, oracle):
    rng = np.random.default_rng(9)
    a = rng.uniform(-1, 1, (6, 10)).astype(np.float32)
    b = rng.uniform(-1, 1, (6, 10)).astype(np.float32)
    zf = ex.exec_pairwise(Pairwise.Subtract, NDArray.from_numpy(a, order="f"), NDArray.from_numpy(b), NDArray.empty((6, 10), FLOAT32, "f"))
    assert np.array_equal(zf.to_numpy(), a - b)
    c = rng.uniform(-1, 1, (3, 4, 2, 5, 6)).astype(np.float32)
    C = NDArray.from_numpy(c)
    perm = (4, 2, 0, 3, 1)
    got = ex.exec_pairwise(Pairwise.Add, C.permute(*perm), C.permute(*perm), NDArray.empty([c.shape[p] for p in perm], FLOAT32))
    assert np.array_equal(got.to_numpy(), 2 * c.transpose(perm))


def test_pairwise_mixed_types_and_type_check(ex, oracle):
    rng = np.random.default_rng(10)
    x = rng.uniform(-1, 1, (5, 7)).astype(np.float32)
    y = rng.uniform(-1, 1, (5, 7)).astype(np.float64)
    z = ex.exec_pairwise(Pairwise.Add, NDArray.from_numpy(x), NDArray.from_numpy(y), NDArray.empty((5, 7), FLOAT32))
    assert np.array_equal(z.to_numpy(), oracle.pairwise(0, x, y, np.zeros_like(x)))
    from deeplearning4j_amd.nativeops import NativeOpsError
    with pytest.raises(NativeOpsError, match="same type as Z"):
        ex.exec_pairwise(Pairwise.Add, NDArray.from_numpy(x), NDArray.from_numpy(x), NDArray.empty((5, 7), DOUBLE))
    with pytest.raises(NativeOpsError, match="equal lengths"):
        ex.exec_pairwise(Pairwise.Add, NDArray.from_numpy(x), NDArray.from_numpy(x[:4]), NDArray.empty((5, 7), FLOAT32))


# ---- transforms ----------------------------------------------------------------------------------------------------
STRICT = [TransformStrict.Tanh, TransformStrict.Sigmoid, TransformStrict.Exp, TransformStrict.Log, TransformStrict.GELU,
          TransformStrict.PreciseGELU, TransformStrict.Swish, TransformStrict.SoftPlus, TransformStrict.Sin, TransformStrict.Cosine,
          TransformStrict.Erf]


@pytest.mark.parametrize("op", STRICT)
@pytest.mark.parametrize("dtype", [FLOAT32, BFLOAT16, HALF, DOUBLE])
def test_transform_strict(ex, oracle, op, dtype):
    rng = np.random.default_rng(200 + op)
    a = rng.uniform(-3, 3, (129, 77))
    if op == TransformStrict.Log:
        a = np.abs(a) + 0.25
    ox, dx = _oracle_arr(oracle, a, dtype)
    oz = _zeros_like(oracle, ox)
    oracle.transform_strict(op, ox, oz)
    got = ex.exec_transform_strict(op, dx)
    rtol, atol = TOL[dtype]
    if dtype == DOUBLE and op in (TransformStrict.Tanh, TransformStrict.PreciseGELU, TransformStrict.Erf):
        rtol, atol = 1e-9, 1e-12     # different exp/pow implementations on the two sides
    gf = got.to_float() if dtype != DOUBLE else got.to_numpy()
    assert_close(gf, _f(oz), rtol, atol, "strict op %d dtype %d" % (op, dtype))


def test_transform_float_and_same(ex, oracle):
    rng = np.random.default_rng(11)
    a = rng.uniform(0.1, 9, (33, 65)).astype(np.float32)
    A = NDArray.from_numpy(a)
    assert np.array_equal(ex.exec_transform_float(TransformFloat.Sqrt, A).to_numpy(), oracle.transform_float(1, a, np.zeros_like(a)))
    assert_close(ex.exec_transform_float(TransformFloat.RSqrt, A).to_numpy(), oracle.transform_float(3, a, np.zeros_like(a)), 2e-7, 0, "rsqrt")
    b = (a - 4).astype(np.float32)
    B = NDArray.from_numpy(b)
    assert np.array_equal(ex.exec_transform_same(TransformSame.Abs, B).to_numpy(), np.abs(b))
    assert np.array_equal(ex.exec_transform_same(TransformSame.Neg, B).to_numpy(), -b)
    assert np.array_equal(ex.exec_transform_same(TransformSame.Square, B).to_numpy(), b * b)
    # Assign converts between types
    z = NDArray.empty(b.shape, DOUBLE)
    ex.exec_assign(B, z)
    assert np.array_equal(z.to_numpy(), b.astype(np.float64))


def test_transform_strided_view(ex, oracle):
    rng = np.random.default_rng(12)
    a = rng.uniform(-2, 2, (16, 12, 24)).astype(np.float32)
    A = NDArray.from_numpy(a)
    got = ex.exec_transform_strict(TransformStrict.Tanh, A.permute(1, 2, 0), NDArray.empty((12, 24, 16), FLOAT32))
    want = oracle.transform_strict(29, a.transpose(1, 2, 0), np.zeros((12, 24, 16), np.float32))
    assert_close(got.to_numpy(), want, 1e-5, 1e-6, "tanh on a permuted view")


def test_transform_strict_rejects_type_change(ex):
    from deeplearning4j_amd.nativeops import NativeOpsError
    with pytest.raises(NativeOpsError, match="same floating point type"):
        ex.exec_transform_strict(TransformStrict.Tanh, NDArray.from_numpy(np.zeros(4, np.float32)), NDArray.empty((4,), DOUBLE))
    with pytest.raises(NativeOpsError, match="not implemented"):
        ex.exec_transform_strict(35, NDArray.from_numpy(np.zeros(4, np.float32)))      # no such opNum in the table
    with pytest.raises(NativeOpsError, match="needs one extra parameter"):
        ex.exec_transform_strict(19, NDArray.from_numpy(np.zeros(4, np.float32)))      # Stabilize without its extraArgs
    with pytest.raises(NativeOpsError, match="needs two extra parameters"):
        ex.exec_transform_strict(2, NDArray.from_numpy(np.zeros(4, np.float32)))       # ScaledTanh without its extraArgs


def test_scalar_and_broadcast(ex, oracle):
    rng = np.random.default_rng(13)
    a = rng.uniform(-1, 1, (9, 20)).astype(np.float32)
    A = NDArray.from_numpy(a)
    assert np.array_equal(ex.exec_scalar(Scalar.Multiply, A, 0.125).to_numpy(), a * np.float32(0.125))
    assert np.array_equal(ex.exec_scalar(Scalar.ReverseSubtract, A, 2.0).to_numpy(), np.float32(2.0) - a)
    row = rng.uniform(-1, 1, 20).astype(np.float32)
    col = rng.uniform(-1, 1, 9).astype(np.float32)
    from deeplearning4j_amd.executioner import Broadcast
    assert np.array_equal(ex.exec_broadcast(Broadcast.Add, A, NDArray.from_numpy(row), [1]).to_numpy(), a + row)
    assert np.array_equal(ex.exec_broadcast(Broadcast.Multiply, A, NDArray.from_numpy(col), [0]).to_numpy(), a * col[:, None])
    assert np.array_equal(ex.exec_broadcast(Broadcast.Add, A, NDArray.from_numpy(row), [1]).to_numpy(), oracle.add_row_vector(a, row, np.zeros_like(a)))


@pytest.mark.parametrize("rows,cols", [(37, 770), (5, 769), (3, 5), (1, 3), (2, 1001), (1000, 7), (65, 4099)])
def test_row_vector_against_rows_of_an_odd_length(ex, rows, cols):
    """A row vector against a dense array whose rows are not whole 16-byte vectors: the array goes as one run of
    element-aligned vectors (the row vector's stretch likewise, element by element across a row's end).  fp32 exactly,
    bf16 as the rounded fp32 result."""
    from deeplearning4j_amd.executioner import Broadcast
    from deeplearning4j_amd.ndarray import BFLOAT16, bf16_bits_to_f32, f32_to_bf16_bits
    rng = np.random.default_rng(rows * 7919 + cols)
    a = rng.uniform(-1, 1, (rows, cols)).astype(np.float32)
    row = rng.uniform(-1, 1, cols).astype(np.float32)
    for op, f in ((Broadcast.Add, np.add), (Broadcast.Multiply, np.multiply), (Broadcast.Subtract, np.subtract)):
        got = ex.exec_broadcast(op, NDArray.from_numpy(a), NDArray.from_numpy(row), [1]).to_numpy()
        assert np.array_equal(got, f(a, row)), (op, rows, cols)
    ab, rb = f32_to_bf16_bits(a), f32_to_bf16_bits(row)
    got = ex.exec_broadcast(Broadcast.Add, NDArray.from_numpy(ab, BFLOAT16), NDArray.from_numpy(rb, BFLOAT16), [1])
    want = f32_to_bf16_bits(bf16_bits_to_f32(ab) + bf16_bits_to_f32(rb))
    assert np.array_equal(f32_to_bf16_bits(got.to_float()), want), (rows, cols)


# ---- reductions ----------------------------------------------------------------------------------------------------------
def _sum_atol(x, axis):
    # |tree sum - sequential sum| <= ~n eps sum|x| in the worst case; sqrt(n)-like in practice
    n = np.prod([x.shape[a] for a in np.atleast_1d(axis)]) if axis is not None else x.size
    return 4 * np.sqrt(n) * EPS32 * np.abs(x.astype(np.float64)).sum(axis).max()


@pytest.mark.parametrize("shape,dims", [((64, 4096), [1]), ((64, 4096), [0]), ((7, 33, 129), [2]), ((7, 33, 129), [0, 1]), ((7, 33, 129), [1]),
                                        ((5, 3, 2, 4, 6), [1, 3]), ((3, 100000), [1]), ((1000, 3), [1])])
def test_reduce_sum_mean_max(ex, oracle, shape, dims):
    rng = np.random.default_rng(300 + len(shape) + dims[0])
    x = rng.uniform(-1, 1, shape).astype(np.float32)
    X = NDArray.from_numpy(x)
    out_shape = [s for i, s in enumerate(shape) if i not in dims]
    atol = _sum_atol(x, tuple(dims))
    got = ex.exec_reduce_same(ReduceSame.Sum, X, dims).to_numpy()
    want = oracle.reduce_same(0, x, np.zeros(out_shape, np.float32), dims)
    assert_close(got, want, 1e-5, atol, "sum %s %s" % (shape, dims))
    assert_close(got, x.astype(np.float64).sum(tuple(dims)), 1e-5, atol, "sum vs fp64")
    n = np.prod([shape[d] for d in dims])
    assert_close(ex.exec_reduce_float(ReduceFloat.Mean, X, dims).to_numpy(), oracle.reduce_float(0, x, np.zeros(out_shape, np.float32), dims), 1e-5, atol / n, "mean")
    assert np.array_equal(ex.exec_reduce_same(ReduceSame.Max, X, dims).to_numpy(), oracle.reduce_same(1, x, np.zeros(out_shape, np.float32), dims))
    assert np.array_equal(ex.exec_reduce_same(ReduceSame.Min, X, dims).to_numpy(), oracle.reduce_same(2, x, np.zeros(out_shape, np.float32), dims))


def test_reduce_full_and_keepdims(ex, oracle):
    rng = np.random.default_rng(14)
    x = rng.uniform(-1, 1, (300, 777)).astype(np.float32)
    X = NDArray.from_numpy(x)
    atol = _sum_atol(x, None)
    assert_close(ex.exec_reduce_same(ReduceSame.Sum, X).to_numpy(), x.astype(np.float64).sum(), 1e-5, atol, "full sum")
    assert_close(ex.exec_reduce_float(ReduceFloat.Mean, X).to_numpy(), x.astype(np.float64).mean(), 1e-5, atol / x.size, "full mean")
    assert ex.exec_reduce_same(ReduceSame.Max, X).to_numpy() == x.max()
    assert_close(ex.exec_reduce_float(ReduceFloat.Norm2, X).to_numpy(), np.sqrt((x.astype(np.float64) ** 2).sum()), 1e-5, 0, "norm2")
    k = ex.exec_reduce_same(ReduceSame.Sum, X, [1], keep_dims=True)
    assert k.shape == (300, 1)
    assert_close(k.to_numpy()[:, 0], x.astype(np.float64).sum(1), 1e-5, _sum_atol(x, 1), "keepdims")
    # strided (permuted) input reduced over what is its last axis
    got = ex.exec_reduce_same(ReduceSame.Sum, X.permute(1, 0), [1]).to_numpy()
    assert_close(got, x.astype(np.float64).sum(0), 1e-5, _sum_atol(x, 0), "permuted")
    # reference vector: Mean of 1..25 = 13, Sum = 325 (NativeOpsTests.cpp:209-238)
    lin = NDArray.from_numpy(np.linspace(1, 25, 25, dtype=np.float32).reshape(5, 5))
    assert ex.exec_reduce_float(ReduceFloat.Mean, lin).to_numpy() == 13
    assert ex.exec_reduce_same(ReduceSame.Sum, lin).to_numpy() == 325


@pytest.mark.parametrize("op", [ReduceSame.Prod, ReduceSame.ASum, ReduceSame.AMax, ReduceSame.AMin])
def test_reduce_same_other_ops(ex, oracle, op):
    rng = np.random.default_rng(op)
    x = (rng.uniform(0.9, 1.1, (50, 40)) * rng.choice([-1, 1], (50, 40))).astype(np.float32)
    got = ex.exec_reduce_same(op, NDArray.from_numpy(x), [1]).to_numpy()
    assert_close(got, oracle.reduce_same(op, x, np.zeros(50, np.float32), [1]), 2e-5, 1e-6, "reduce_same %d" % op)


@pytest.mark.parametrize("op", [ReduceFloat.AMean, ReduceFloat.Norm1, ReduceFloat.Norm2, ReduceFloat.NormMax, ReduceFloat.SquaredNorm])
def test_reduce_float_other_ops(ex, oracle, op):
    rng = np.random.default_rng(op)
    x = rng.normal(0, 1, (40, 300)).astype(np.float32)
    got = ex.exec_reduce_float(op, NDArray.from_numpy(x), [1]).to_numpy()
    assert_close(got, oracle.reduce_float(op, x, np.zeros(40, np.float32), [1]), 2e-5, 1e-5, "reduce_float %d" % op)


@pytest.mark.parametrize("dtype", [BFLOAT16, HALF])
def test_reduce_half_types_accumulate_in_float(ex, oracle, dtype):
    rng = np.random.default_rng(15)
    a = rng.uniform(-1, 1, (32, 2048))
    ox, dx = _oracle_arr(oracle, a, dtype)
    oz = oracle.Arr(np.zeros(32, ox.a.dtype), ox.dt)
    oracle.reduce_same(0, ox, oz, [1])
    got = ex.exec_reduce_same(ReduceSame.Sum, dx, [1]).to_float()
    assert_close(got, _f(oz), 1e-2, 1e-2, "half sum")


# ---- index reductions: bit-exact ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("shape,dims", [((64, 4096), [1]), ((64, 4096), [0]), ((9, 17, 33), [2]), ((9, 17, 33), [1]), ((9, 17, 33), [0, 2]),
                                        ((4, 50257), [1]), ((2000, 5), [1]), ((1, 300000), [1])])
@pytest.mark.parametrize("op", [IndexReduce.IndexMax, IndexReduce.IndexMin])
def test_index_reduce_bit_exact(ex, oracle, shape, dims, op):
    rng = np.random.default_rng(400 + shape[0] + op)
    x = rng.uniform(-1, 1, shape).astype(np.float32)
    out_shape = [s for i, s in enumerate(shape) if i not in dims]
    want = oracle.index_reduce(op, x, np.zeros(out_shape, np.int64), dims)
    got = ex.exec_index_reduce(op, NDArray.from_numpy(x), dims).to_numpy()
    assert got.dtype == np.int64 and np.array_equal(got, want)


def test_index_reduce_ties_nan_inf_and_scalar(ex, oracle):
    rng = np.random.default_rng(16)
    x = rng.integers(-2, 3, (300, 1000)).astype(np.float32)          # heavy ties: the first extreme must win
    for op in (0, 1, 2, 3):
        want = oracle.index_reduce(op, x, np.zeros(300, np.int64), [1])
        assert np.array_equal(ex.exec_index_reduce(op, NDArray.from_numpy(x), [1]).to_numpy(), want), op
    inf, nan = np.inf, np.nan
    rows = np.array([[1, 3, 3, 2], [nan, 1, 2, 2], [-inf, -inf, -inf, -inf], [nan, nan, nan, nan], [nan, -inf, 5, nan], [2, 2, 2, 2]], np.float32)
    rows = np.tile(rows, (1, 700))                                      # long rows: cooperative path
    for op in (0, 1, 2, 3):
        want = oracle.index_reduce(op, rows, np.zeros(6, np.int64), [1])
        assert np.array_equal(ex.exec_index_reduce(op, NDArray.from_numpy(rows), [1]).to_numpy(), want), op
    # reference vectors: NativeOpsTests.cpp:84-117, LegacyOpsTests.cpp:279-310
    lin = np.linspace(1, 25, 25, dtype=np.float32).reshape(5, 5)
    assert ex.exec_index_reduce(0, NDArray.from_numpy(lin)).to_numpy() == 24
    assert list(ex.exec_index_reduce(0, NDArray.from_numpy(lin), [1]).to_numpy()) == [4] * 5
    z32 = NDArray.empty((5,), INT32)
    ex.exec_index_reduce(0, NDArray.from_numpy(lin), [1], z=z32)
    assert list(z32.to_numpy()) == [4] * 5
    big = rng.uniform(-1, 1, 3_000_001).astype(np.float32)
    big[[123456, 2999999]] = 2.0
    assert ex.exec_index_reduce(0, NDArray.from_numpy(big)).to_numpy() == 123456


@pytest.mark.parametrize("dtype", [FLOAT32, BFLOAT16, HALF, DOUBLE])
@pytest.mark.parametrize("rows,L,first", [(32, 50257, 0), (1, 50257, 3), (4, 200003, 1), (7, 3001, 5), (3, 17, 1), (2, 40001, 7)])
def test_index_reduce_rows_that_start_off_a_16_byte_boundary(ex, oracle, dtype, rows, L, first):
    """Rows of an odd length, and the columns first.. of a wider matrix: no row starts on a 16-byte boundary, so a run is
    read as a scalar head, vectors and a scalar tail (cut into segments where the rows are few and long).  Heavy ties, and
    rows whose only extreme sits in the head, in the last element, or on both sides of a segment boundary."""
    rng = np.random.default_rng(rows * L + first)
    full = rng.integers(-3, 4, (rows, L + first)).astype(np.float64)
    x = full[:, first:]
    x[0, :] = 1.0                                   # all equal: index 0
    if rows > 1: x[1, :] = -3.0; x[1, 0] = 5.0; x[1, L - 1] = -5.0          # extremes in the head and in the last element
    if rows > 2: x[2, :] = 0.0; x[2, L - 1] = 4.0; x[2, 1] = -4.0
    if rows > 3 and L > 8448 + 2: x[3, :] = 0.0; x[3, [8447, 8448, 8449]] = 2.0    # a tie across a segment boundary
    _, dfull = _oracle_arr(oracle, full, dtype)     # small integers: exact in every storage type
    dx = dfull.slice(1, first, first + L) if first else dfull
    xr = np.ascontiguousarray(x).astype(np.float64 if dtype == DOUBLE else np.float32)
    for op in (0, 1, 2, 3):
        want = oracle.index_reduce(op, xr, np.zeros(rows, np.int64), [1])
        assert np.array_equal(ex.exec_index_reduce(op, dx, [1]).to_numpy(), want), (op, rows, L, first)
    assert np.array_equal(ex.exec_index_reduce(0, dx, [1]).to_numpy(), xr.argmax(1))


@pytest.mark.parametrize("dtype", [FLOAT32, BFLOAT16, HALF, DOUBLE])
@pytest.mark.parametrize("rows,cols,first,width", [(6144, 512, 0, 512), (1000, 4096, 0, 4096), (777, 1001, 0, 1001), (4100, 96, 3, 128), (300, 64, 0, 64),
                                                   (9, 2048, 0, 2048), (40000, 17, 0, 17)])
def test_reductions_down_the_columns(ex, oracle, dtype, rows, cols, first, width):
    """Reductions over dim 0 of a row-major matrix (the outputs lie side by side, the reduced axis walks at the row pitch):
    many rows cut over several blocks, few rows, an odd column count, columns first.. of a wider matrix (rows at a pitch, starts
    off the 4-byte pairs of the 16-bit types).  Sums within the re-ordered-sum bound, extremes exact; also the leading two dims
    of a rank-3 array."""
    rng = np.random.default_rng(rows + cols + first)
    full = rng.uniform(-1, 1, (rows, width))
    _, dfull = _oracle_arr(oracle, full, dtype)
    X = dfull.slice(1, first, first + cols) if width != cols else dfull
    held = dfull.to_float().astype(np.float64)[:, first:first + cols]
    tol = {FLOAT32: 1e-5, DOUBLE: 1e-12, BFLOAT16: 1e-2, HALF: 2e-3}[dtype]
    atol = _sum_atol(held.astype(np.float32), 0) if dtype == FLOAT32 else tol * np.abs(held).sum(0).max()
    got = ex.exec_reduce_same(ReduceSame.Sum, X, [0]).to_float().astype(np.float64)
    assert_close(got, held.sum(0), tol, atol, "sum down the columns")
    got = ex.exec_reduce_float(ReduceFloat.Mean, X, [0]).to_float().astype(np.float64)
    assert_close(got, held.mean(0), tol, atol / rows + tol * 1e-3, "mean down the columns")
    got = ex.exec_reduce_float(ReduceFloat.Norm2, X, [0]).to_float().astype(np.float64)
    assert_close(got, np.sqrt((held ** 2).sum(0)), 2 * tol, 0, "norm2 down the columns")
    assert np.array_equal(ex.exec_reduce_same(ReduceSame.Max, X, [0]).to_float().astype(np.float64), held.max(0))
    assert np.array_equal(ex.exec_reduce_same(ReduceSame.Min, X, [0]).to_float().astype(np.float64), held.min(0))
    if width == cols and rows % 4 == 0:
        X3 = dfull.reshape(4, rows // 4, cols)
        got = ex.exec_reduce_same(ReduceSame.Sum, X3, [0, 1]).to_float().astype(np.float64)
        assert_close(got, held.sum(0), tol, atol, "sum over the two leading dims")


@pytest.mark.parametrize("dtype", [FLOAT32, BFLOAT16, HALF, DOUBLE])
@pytest.mark.parametrize("rows,cols,first,width", [(6144, 512, 0, 512), (777, 1001, 0, 1001), (4100, 96, 3, 128), (9, 2048, 0, 2048), (40000, 17, 0, 17)])
def test_index_reductions_down_the_columns(ex, oracle, dtype, rows, cols, first, width):
    """IndexMax / IndexMin / IndexAbsoluteMax / IndexAbsoluteMin over dim 0 of a row-major matrix: heavy ties (the first row
    with the extreme wins, whichever wave or block met it), an all-equal column, NaN never selected; dense, an odd column
    count, and the columns first.. of a wider matrix."""
    rng = np.random.default_rng(rows * 3 + cols + first)
    full = rng.integers(-3, 4, (rows, width)).astype(np.float64)
    full[:, first] = 1.0                                         # an all-equal column: row 0
    full[rows - 1, first + 1] = 9.0                              # the extreme in the last row
    if dtype != DOUBLE:
        full[rows // 2, first + 2] = np.nan
    _, dfull = _oracle_arr(oracle, full, dtype)
    X = dfull.slice(1, first, first + cols) if width != cols else dfull
    x = np.ascontiguousarray(full[:, first:first + cols]).astype(np.float64 if dtype == DOUBLE else np.float32)
    for op in (0, 1, 2, 3):
        want = oracle.index_reduce(op, x, np.zeros(cols, np.int64), [0])
        assert np.array_equal(ex.exec_index_reduce(op, X, [0]).to_numpy(), want), (op, rows, cols)


@pytest.mark.parametrize("rows,L,pitch", [(37, 1028, 1028), (5, 8192, 8192), (9, 5000, 5000), (33, 4096, 4352), (3, 1024, 2048)])
def test_reductions_over_rows_at_a_constant_pitch(ex, oracle, rows, L, pitch):
    """Rows of 1024..8192 elements at a constant pitch take the one-shot kernels (all loads up front, masked tail):
    value reductions within the re-ordered-sum bound, index reductions bit-exact, also on a column slice of a wider
    matrix."""
    rng = np.random.default_rng(rows + L)
    wide = rng.uniform(-1, 1, (rows, pitch)).astype(np.float32)
    wide[:, L // 2] = 1.5
    wide[: rows // 2, L - 1] = 1.5                      # a tie with the last element of the row
    x = np.ascontiguousarray(wide[:, :L])
    X = NDArray.from_numpy(wide).view((rows, L), (pitch, 1), 0)
    atol = _sum_atol(x, 1)
    assert_close(ex.exec_reduce_same(ReduceSame.Sum, X, [1]).to_numpy(), oracle.reduce_same(0, x, np.zeros(rows, np.float32), [1]), 1e-5, atol, "sum")
    assert_close(ex.exec_reduce_float(ReduceFloat.Mean, X, [1]).to_numpy(), x.astype(np.float64).mean(1), 1e-5, atol / L, "mean")
    assert_close(ex.exec_reduce_float(ReduceFloat.Norm2, X, [1]).to_numpy(), np.sqrt((x.astype(np.float64) ** 2).sum(1)), 1e-5, 0, "norm2")
    assert np.array_equal(ex.exec_reduce_same(ReduceSame.Max, X, [1]).to_numpy(), x.max(1))
    assert np.array_equal(ex.exec_reduce_same(ReduceSame.Min, X, [1]).to_numpy(), x.min(1))
    for op in (0, 1, 2, 3):
        want = oracle.index_reduce(op, x, np.zeros(rows, np.int64), [1])
        assert np.array_equal(ex.exec_index_reduce(op, X, [1]).to_numpy(), want), op
    assert list(ex.exec_index_reduce(0, X, [1]).to_numpy()) == [L // 2] * rows


@pytest.mark.parametrize("dtype", [BFLOAT16, HALF])
def test_index_reduce_half_types(ex, oracle, dtype):
    rng = np.random.default_rng(17)
    a = rng.uniform(-1, 1, (50, 3000))
    ox, dx = _oracle_arr(oracle, a, dtype)   # rounding creates ties; the comparison happens on the rounded values
    want = oracle.index_reduce(0, ox, np.zeros(50, np.int64), [1])
    assert np.array_equal(ex.exec_index_reduce(0, dx, [1]).to_numpy(), want)


# ---- BASELINE config 1 at full size: size-independent properties ---------------------------------------------------------------
def test_config1_chain_full_size(ex, oracle):
    """fp32 [8192, 4096]: add -> tanh -> reduce_sum(dim 1) -> argmax(dim 1); the oracle checks a row sample,
    the rest is covered by properties that hold at any size."""
    rng = np.random.default_rng(1001)
    x = rng.uniform(-1, 1, (8192, 4096)).astype(np.float32)
    y = rng.uniform(-1, 1, (8192, 4096)).astype(np.float32)
    X, Y = NDArray.from_numpy(x), NDArray.from_numpy(y)
    S = ex.exec_pairwise(Pairwise.Add, X, Y)
    T = ex.exec_transform_strict(TransformStrict.Tanh, S)
    R = ex.exec_reduce_same(ReduceSame.Sum, T, [1])
    A = ex.exec_index_reduce(IndexReduce.IndexMax, T, [1])
    s, t, r, a = S.to_numpy(), T.to_numpy(), R.to_numpy(), A.to_numpy()
    assert np.array_equal(s, x + y)                                              # exact everywhere
    rows = rng.choice(8192, 64, replace=False)
    want_t = oracle.transform_strict(29, s[rows], np.zeros((64, 4096), np.float32))
    assert_close(t[rows], want_t, 1e-5, 1e-6, "tanh sample")
    assert np.abs(t).max() <= 1.0 and (np.sign(t) == np.sign(s)).all()               # odd, bounded
    assert_close(r, t.astype(np.float64).sum(1), 1e-5, 4 * 64 * EPS32 * np.abs(t).sum(1).max(), "row sums")
    assert np.array_equal(a, np.argmax(t, axis=1))                                # first maximum, every row
    assert np.array_equal(a[rows], oracle.index_reduce(0, t[rows], np.zeros(64, np.int64), [1]))
