"""The bool tables through the C ABI (execPairwiseTransformBool, execScalarBool, execBroadcastBool, execScalarBoolTad) and
execScalarTad: the reference's own test vectors, then every op of the tables over every operand type against the oracle's
restatement, on dense arrays, views and broadcast operands.  BOOL results: the comparison is exact."""
import numpy as np
import pytest

from deeplearning4j_amd import nativeops as N
from deeplearning4j_amd.executioner import BoolOp, Scalar
from deeplearning4j_amd.ndarray import BFLOAT16, BOOL, DOUBLE, FLOAT32, HALF, INT32, INT64, NDArray, bf16_bits_to_f32, f32_to_bf16_bits

pytestmark = pytest.mark.gpu

OPS = [BoolOp.EqualTo, BoolOp.GreaterThan, BoolOp.LessThan, BoolOp.Epsilon, BoolOp.GreaterThanOrEqual, BoolOp.NotEqualTo, BoolOp.And, BoolOp.Or,
       BoolOp.Xor, BoolOp.Not, BoolOp.LessThanOrEqual]
NP = {DOUBLE: np.float64, FLOAT32: np.float32, HALF: np.float16, INT32: np.int32, INT64: np.int64, BOOL: np.bool_}


def _values(rng, shape, dt):
    """Small integers with many ties and zeros, pairs that differ by less than the default tolerance, NaN for the float types."""
    v = rng.integers(-2, 3, shape).astype(np.float64)
    if dt == BOOL:
        return (v > 0), NDArray.from_numpy(v > 0)
    if dt in (INT32, INT64):
        a = v.astype(NP[dt])
        return a, NDArray.from_numpy(a)
    flat = v.reshape(-1)
    flat[::7] += 4e-6
    flat[3::11] += 0.5
    if flat.size > 20:
        flat[5::13] = np.nan
    if dt == BFLOAT16:
        held = bf16_bits_to_f32(f32_to_bf16_bits(v.astype(np.float32)))
        return held, NDArray.from_numpy(held, BFLOAT16)
    a = v.astype(NP[dt])
    return a, NDArray.from_numpy(a)


def _want(oracle, op, x, y, dt, params=None):
    return oracle.bool_table(op, x, y, params, bf16=(dt == BFLOAT16))


def test_reference_vectors(ex, oracle):
    # MultiDataTypeTests.cpp:1095-1124: one length, different shapes
    x1, x2 = NDArray.from_numpy(np.array([[1, 1, 2], [3, 4, 5]], np.int32)), NDArray.from_numpy(np.array([[1, 0], [2, 0], [4, 0]], np.int32))
    z = NDArray.empty((3, 2), BOOL)
    assert ex.exec_pairwise_bool(BoolOp.EqualTo, x1, x2, z=z).to_numpy().reshape(-1).tolist() == [1, 0, 1, 0, 1, 0]
    x3, x4 = NDArray.from_numpy(np.array([[0.5, 1.5], [2.5, 3], [4.5, 0]])), NDArray.from_numpy(np.array([[0.5, 1., 2.5], [3, 4., 0]]))
    assert ex.exec_pairwise_bool(BoolOp.EqualTo, x3, x4, z=NDArray.empty((2, 3), BOOL)).to_numpy().reshape(-1).tolist() == [1, 0, 1, 1, 0, 1]
    x5, x6 = NDArray.from_numpy(np.array([[0, 1], [0, 1], [0, 1]], bool)), NDArray.from_numpy(np.array([[1, 1, 1], [0, 1, 0]], bool))
    assert ex.exec_pairwise_bool(BoolOp.EqualTo, x5, x6, z=NDArray.empty((2, 3), BOOL)).to_numpy().reshape(-1).tolist() == [0, 1, 0, 0, 0, 0]
    # MultiDataTypeTests.cpp:1150-1172: broadcast along dimension 0
    b1, b2 = NDArray.from_numpy(np.array([[10, 20, 30], [40, 50, 60]], np.int32)), NDArray.from_numpy(np.array([10, 60], np.int32))
    assert ex.exec_broadcast_bool(BoolOp.EqualTo, b1, b2, [0]).to_numpy().reshape(-1).tolist() == [1, 0, 0, 0, 0, 1]
    b4, b5 = NDArray.from_numpy(np.array([[0, 0, 0], [0, 0, 1]], bool)), NDArray.from_numpy(np.array([0, 1], bool))
    assert ex.exec_broadcast_bool(BoolOp.EqualTo, b4, b5, [0]).to_numpy().reshape(-1).tolist() == [1, 1, 1, 0, 0, 1]
    # MultiDataTypeTests.cpp:1290-1311: scalars
    assert ex.exec_scalar_bool(BoolOp.EqualTo, NDArray.from_numpy(np.array([[0, 1], [2, 3]], np.int64)), 1).to_numpy().reshape(-1).tolist() == [0, 1, 0, 0]
    assert ex.exec_scalar_bool(BoolOp.EqualTo, NDArray.from_numpy(np.array([[0, 1.5], [2.5, 3.5]], np.float32)), 1.5).to_numpy().reshape(-1).tolist() == [0, 1, 0, 0]
    assert ex.exec_scalar_bool(BoolOp.EqualTo, NDArray.from_numpy(np.array([[0, 1], [1, 0]], bool)), True).to_numpy().reshape(-1).tolist() == [0, 1, 1, 0]
    # NativeOpsTests.cpp:144-167 (ExecBroadcast_2), :186-206 (ExecPairwise_2), :565-585 (scalar GreaterThan)
    lin = np.arange(1, 26, dtype=np.float32).reshape(5, 5)
    z = ex.exec_broadcast_bool(BoolOp.EqualTo, NDArray.from_numpy(lin), NDArray.from_numpy(np.arange(2, 11, 2, dtype=np.float32).reshape(5, 1)), [0]).to_numpy().reshape(-1)
    assert z[1] and not z[0]
    y = np.zeros((5, 5), bool); y.reshape(-1)[5] = True
    z = ex.exec_pairwise_bool(BoolOp.And, NDArray.from_numpy(np.ones((5, 5), bool)), NDArray.from_numpy(y)).to_numpy().reshape(-1)
    assert z[5] and not z[4]
    z = ex.exec_scalar_bool(BoolOp.GreaterThan, NDArray.from_numpy(lin), 10.0).to_numpy().reshape(-1)
    assert not z[5] and z[15] and np.array_equal(z, lin.reshape(-1) > 10)
    # NativeOpsTests.cpp:762-793 (ScalarTadTest_1): Multiply by one scalar, dimensions 0 and 1; :803-832 (ScalarTadTest_2): And
    got = ex.exec_scalar_tad(Scalar.Multiply, NDArray.from_numpy(lin), NDArray.from_numpy(np.array(10.0, np.float32)), [0, 1]).to_numpy()
    assert np.array_equal(got, np.arange(10, 260, 10, dtype=np.float32).reshape(5, 5))
    xb = np.zeros((5, 5), bool); xb.reshape(-1)[[5, 15]] = True
    z = ex.exec_scalar_bool_tad(BoolOp.And, NDArray.from_numpy(xb), NDArray.from_numpy(np.array(True)), [0, 1]).to_numpy().reshape(-1)
    assert z[5] and z[15] and z.sum() == 2


@pytest.mark.parametrize("dt", [FLOAT32, DOUBLE, HALF, BFLOAT16, INT32, INT64, BOOL])
@pytest.mark.parametrize("op", OPS)
def test_pairwise_and_scalar_against_the_oracle(ex, oracle, dt, op):
    rng = np.random.default_rng(100 * op + dt)
    shape = (37, 53)
    x, X = _values(rng, shape, dt)
    y, Y = _values(rng, shape, dt)
    assert np.array_equal(ex.exec_pairwise_bool(op, X, Y).to_numpy(), _want(oracle, op, x, y, dt)), "dense"
    # a transposed view against a dense array, into a column slice of a wider result
    xt, Xt = _values(rng, (53, 37), dt)
    wide = NDArray.from_numpy(np.ones((37, 60), bool))
    ex.exec_pairwise_bool(op, Xt.permute(1, 0), Y, z=wide.slice(1, 4, 57))
    w = wide.to_numpy()
    assert np.array_equal(w[:, 4:57], _want(oracle, op, np.ascontiguousarray(xt.T), y, dt)) and w[:, :4].all() and w[:, 57:].all(), "views"
    # a one-element y stands for a scalar; execScalarBool takes the same value
    for s in (1, 0, -2) if dt != BOOL else (True, False):
        sv = np.full(shape, s, x.dtype)
        want = _want(oracle, op, x, sv, dt)
        S = NDArray.scalar(s, dt)
        assert np.array_equal(ex.exec_pairwise_bool(op, X, S).to_numpy(), want), ("pairwise with a scalar y", s)
        assert np.array_equal(ex.exec_scalar_bool(op, X, S).to_numpy(), want), ("scalar", s)
    # the ops that read a parameter
    if op in (BoolOp.Epsilon, BoolOp.And, BoolOp.Or, BoolOp.Xor):
        for p0 in ((0.5, 1.0) if op == BoolOp.Epsilon else (1.0, 0.0)):
            got = ex.exec_pairwise_bool(op, X, Y, extra_args=[p0]).to_numpy()
            assert np.array_equal(got, _want(oracle, op, x, y, dt, [p0])), ("parameter", p0)


@pytest.mark.parametrize("dt", [FLOAT32, BFLOAT16, INT32, BOOL])
@pytest.mark.parametrize("op", [BoolOp.EqualTo, BoolOp.LessThan, BoolOp.Epsilon, BoolOp.And, BoolOp.Xor, BoolOp.Not, BoolOp.GreaterThanOrEqual])
def test_broadcast_and_per_sub_array_scalars_against_the_oracle(ex, oracle, dt, op):
    rng = np.random.default_rng(7 * op + dt)
    shape = (3, 5, 4, 6)
    x, X = _values(rng, shape, dt)
    for dims, yshape in (([3], (6,)), ([1], (5,)), ([0, 2], (3, 4)), ([1, 2, 3], (5, 4, 6)), ([0, 3], (3, 1, 6))):
        y, Y = _values(rng, yshape, dt)
        want = _want(oracle, op, x, np.ascontiguousarray(oracle.operand_along(y, shape, dims)), dt)
        assert np.array_equal(ex.exec_broadcast_bool(op, X, Y, dims).to_numpy(), want), dims
    # DeclarableOpsTests9.cpp:811-834 (test_broadcast_bool_1 / _2): unit dims on both sides, y a slice of a larger array
    x5, X5 = _values(rng, (1, 3, 2, 4, 4), dt)
    o, Orig = _values(rng, (1, 7, 4, 4), dt)
    Ys = Orig.slice(1, 2, 4)
    want = _want(oracle, op, x5, np.ascontiguousarray(oracle.operand_along(o[:, 2:4], x5.shape, [0, 2, 3, 4])), dt)
    assert np.array_equal(ex.exec_broadcast_bool(op, X5, Ys, [0, 2, 3, 4]).to_numpy(), want)
    # one scalar per sub-array along dims
    for dims in ([3], [1, 2], [0], [0, 1, 2, 3]):
        n = int(np.prod([shape[d] for d in range(4) if d not in dims])) if len(dims) < 4 else 1
        s, S = _values(rng, (n,), dt)
        want = _want(oracle, op, x, np.ascontiguousarray(oracle.scalars_along(s, shape, dims)), dt)
        assert np.array_equal(ex.exec_scalar_bool_tad(op, X, S, dims).to_numpy(), want), dims


@pytest.mark.parametrize("dt", [FLOAT32, BFLOAT16, INT64])
def test_scalar_tad_is_execscalar_per_sub_array(ex, dt):
    """execScalarTad against execScalar applied to each sub-array with its own scalar (the same kernels' arithmetic, so
    the comparison is exact), rows and columns of a matrix and planes of a rank-3 array."""
    rng = np.random.default_rng(dt)
    x = rng.integers(-5, 6, (6, 7, 4))
    X = NDArray.from_numpy(x.astype(np.float32), dt) if dt != INT64 else NDArray.from_numpy(x.astype(np.int64))
    for op in (Scalar.Add, Scalar.Multiply, Scalar.ReverseSubtract, Scalar.MaxPairwise):
        for dims in ([2], [0, 1], [1]):
            other = [d for d in range(3) if d not in dims]
            n = int(np.prod([x.shape[d] for d in other]))
            sv = rng.integers(-3, 4, n)
            S = NDArray.from_numpy(sv.astype(np.float32), dt) if dt != INT64 else NDArray.from_numpy(sv.astype(np.int64))
            got = ex.exec_scalar_tad(op, X, S, dims).to_numpy()
            xf, sf = x.astype(np.float64), oracle_free_scalars(sv, x.shape, dims)
            want = {Scalar.Add: xf + sf, Scalar.Multiply: xf * sf, Scalar.ReverseSubtract: sf - xf, Scalar.MaxPairwise: np.maximum(xf, sf)}[op]
            gotf = bf16_bits_to_f32(got).astype(np.float64) if dt == BFLOAT16 else got.astype(np.float64)
            assert np.array_equal(gotf, want), (op, dims)       # small integers: exact in every type


def oracle_free_scalars(s, x_shape, dims):
    """numpy only: scalar r belongs to the r-th sub-array in c order over the dims outside `dims`."""
    other = [d for d in range(len(x_shape)) if d not in dims]
    full = [x_shape[d] if d in other else 1 for d in range(len(x_shape))]
    return np.broadcast_to(np.asarray(s, np.float64).reshape(full), x_shape)


def test_errors(ex):
    L = ex.L
    x, y = NDArray.from_numpy(np.ones((4, 4), np.float32)), NDArray.from_numpy(np.ones((4, 4), np.float32))
    with pytest.raises(N.NativeOpsError, match="BOOL"):
        ex.exec_pairwise_bool(BoolOp.EqualTo, x, y, z=NDArray.empty((4, 4), FLOAT32))
    with pytest.raises(N.NativeOpsError, match="one type"):
        ex.exec_pairwise_bool(BoolOp.EqualTo, x, NDArray.from_numpy(np.ones((4, 4), np.int32)))
    with pytest.raises(N.NativeOpsError, match="opNum 5"):
        ex.exec_pairwise_bool(BoolOp.MatchCondition, x, y)
    with pytest.raises(N.NativeOpsError, match="one length"):
        ex.exec_pairwise_bool(BoolOp.EqualTo, x, NDArray.from_numpy(np.ones((4, 3), np.float32)))
    with pytest.raises(N.NativeOpsError, match="scalars for"):
        ex.exec_scalar_bool_tad(BoolOp.EqualTo, x, NDArray.from_numpy(np.ones(3, np.float32)), [1])
    with pytest.raises(N.NativeOpsError, match="does not match"):
        ex.exec_broadcast_bool(BoolOp.EqualTo, x, NDArray.from_numpy(np.ones(3, np.float32)), [1])
    assert L.lastErrorCode() == 0


# ---- execReduce3All: every sub-array of x against every sub-array of y ----------------------------------------------------
def test_reduce3_all_reference_vectors(ex):
    from deeplearning4j_amd.executioner import Reduce3
    x, y = NDArray.from_numpy(np.array([[1, 2, 3], [4, 5, 6]], np.float32)), NDArray.from_numpy(np.full((2, 3), 2, np.float32))
    got = ex.exec_reduce3_all(Reduce3.EuclideanDistance, x, y, [1]).to_numpy()                     # NDArrayTests.cpp:1455-1470
    np.testing.assert_allclose(got, [[1.414214, 1.414214], [5.385165, 5.385165]], rtol=1e-6)
    c = NDArray.from_numpy(np.array([[1, 2, 3], [2, 3, 4]], np.float64))
    np.testing.assert_allclose(ex.exec_reduce3_all(Reduce3.EuclideanDistance, c, c, [1]).to_numpy(), [[0, 1.73205], [1.73205, 0]], rtol=1e-5)   # NDArrayTests2.cpp:199-209
    x4, x3 = NDArray.from_numpy(np.array([[1, 2], [3, 4]], np.float64)), NDArray.from_numpy(np.full((2, 3), 1.5))
    assert np.array_equal(ex.exec_reduce3_all(Reduce3.Dot, x4, x3, [0]).to_numpy(), [[6, 6, 6], [9, 9, 9]])        # MultiDataTypeTests.cpp:1629-1644


@pytest.mark.parametrize("dt,tol", [(FLOAT32, 1e-5), (DOUBLE, 1e-12), (BFLOAT16, 1e-2), (HALF, 2e-3)])
def test_reduce3_all_against_the_oracle(ex, oracle, dt, tol):
    from conftest import assert_close
    from deeplearning4j_amd.executioner import Reduce3
    rng = np.random.default_rng(dt)

    def held(a):
        if dt == BFLOAT16:
            return bf16_bits_to_f32(f32_to_bf16_bits(a.astype(np.float32))).astype(np.float64)
        return a.astype(NP[dt]).astype(np.float64)

    def out(z):
        return bf16_bits_to_f32(z).astype(np.float64) if dt == BFLOAT16 else z.astype(np.float64)

    for xs, ys, dims in (((5, 33), (7, 33), [1]), ((40, 6), (40, 3), [0]), ((2, 9, 3, 5), (3, 9, 2, 5), [1, 3]), ((4, 300), (4, 300), [1])):
        x, y = held(rng.normal(0, 1, xs)), held(rng.normal(0, 1, ys))
        X = NDArray.from_numpy(x.astype(np.float32), dt) if dt == BFLOAT16 else NDArray.from_numpy(x.astype(NP[dt]))
        Y = NDArray.from_numpy(y.astype(np.float32), dt) if dt == BFLOAT16 else NDArray.from_numpy(y.astype(NP[dt]))
        for op in (Reduce3.ManhattanDistance, Reduce3.EuclideanDistance, Reduce3.CosineSimilarity, Reduce3.Dot, Reduce3.CosineDistance):
            want = oracle.reduce3_all(op, x, y, dims)                    # the oracle in float64 on the values the arrays hold
            got = out(ex.exec_reduce3_all(op, X, Y, dims).to_numpy())
            scale = max(1.0, float(np.abs(want).max()))
            assert_close(got, want, tol, tol * scale, "reduce3 all-pairs op %d %s %s" % (op, xs, dims))
    # the result may be a view: columns 2.. of a wider matrix
    x, y = held(rng.normal(0, 1, (5, 16))), held(rng.normal(0, 1, (6, 16)))
    X = NDArray.from_numpy(x.astype(np.float32), dt) if dt == BFLOAT16 else NDArray.from_numpy(x.astype(NP[dt]))
    Y = NDArray.from_numpy(y.astype(np.float32), dt) if dt == BFLOAT16 else NDArray.from_numpy(y.astype(NP[dt]))
    wide = NDArray.from_numpy(np.zeros((5, 10), np.float32), dt) if dt == BFLOAT16 else NDArray.from_numpy(np.zeros((5, 10), NP[dt]))
    ex.exec_reduce3_all(Reduce3.Dot, X, Y, [1], z=wide.slice(1, 2, 8))
    w = out(wide.to_numpy())
    assert_close(w[:, 2:8], x @ y.T, tol, tol * 8, "into a view")
    assert not w[:, :2].any() and not w[:, 8:].any()
