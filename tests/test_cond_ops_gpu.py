"""The legacy ops that read a match condition, an exponent or a tolerance from extraParams, through the C ABI, against the
numpy restatements in oracle/oracle.py (pinned to the reference's own vectors in tests/test_oracle_cond_ops.py) and against
those vectors directly (libnd4j/tests_cpu/layers_tests/NDArrayTests2.cpp:96-103; platform-tests
.../nd4j/linalg/indexing/BooleanIndexingTest.java:208-335).  Elementwise results and counts / positions are exact."""
import numpy as np
import pytest

from deeplearning4j_amd.executioner import IndexReduce, Pairwise, Reduce3, ReduceFloat, ReduceLong, Scalar, TransformBool, TransformSame
from deeplearning4j_amd.ndarray import BFLOAT16, DOUBLE, FLOAT32, HALF, INT32, INT64, NDArray
from oracle import oracle as O

pytestmark = pytest.mark.gpu

EPS = 1e-5
NP = {FLOAT32: np.float32, DOUBLE: np.float64, HALF: np.float16, INT32: np.int32, INT64: np.int64}
FLOATS = [FLOAT32, DOUBLE, HALF]
MODES = list(range(16))


def _draw(rng, shape, dt, special=True):
    """Halves in [-4, 4] (so that ==, <= and the eps modes all hit) with a few inf / nan among the floating types."""
    if dt in (INT32, INT64):
        return rng.integers(-4, 5, shape).astype(NP[dt])
    a = (rng.integers(-8, 9, shape) / 2.0).astype(NP[dt])
    if special:
        flat = a.reshape(-1)
        pick = rng.choice(flat.size, max(1, flat.size // 37), replace=False)
        flat[pick] = rng.choice(np.array([np.inf, -np.inf, np.nan]), pick.size).astype(NP[dt])
    return a


def _same(got, want):
    return np.array_equal(got, want, equal_nan=np.asarray(want).dtype.kind == "f")


@pytest.mark.parametrize("dt", FLOATS + [INT32, INT64])
@pytest.mark.parametrize("mode", MODES)
def test_match_condition_bool_and_compare_and_set_transform(ex, dt, mode):
    rng = np.random.default_rng(100 + mode + 16 * dt)
    x = _draw(rng, (67, 131), dt)
    compare, eps = (1.0, 1.0) if dt in (INT32, INT64) else (1.0, 0.5)
    X = NDArray.from_numpy(x)
    got = ex.exec_transform_bool(TransformBool.MatchConditionBool, X, extra_args=[compare, eps, mode]).to_numpy()
    assert np.array_equal(got, O.match_mask(x, compare, eps, mode))
    if dt != INT64:   # the value-carrying ops stop at INT32 (see test_int64_values_are_refused)
        got = ex.exec_transform_same(TransformSame.CompareAndSetTransform, X, extra_args=[compare, 7.0, eps, mode]).to_numpy()
        assert _same(got, O.compare_and_set_transform(x, compare, 7.0, eps, mode))
    # a permuted view of the same values
    Xt = NDArray.from_numpy(np.ascontiguousarray(x.T)).permute(1, 0)
    got = ex.exec_transform_bool(TransformBool.MatchConditionBool, Xt, extra_args=[compare, eps, mode]).to_numpy()
    assert np.array_equal(got, O.match_mask(x, compare, eps, mode))


@pytest.mark.parametrize("mode", [2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15])
def test_match_condition_bfloat16(ex, mode):
    rng = np.random.default_rng(mode)
    x = _draw(rng, (33, 65), FLOAT32)                       # halves are exact in bfloat16
    X = NDArray.from_numpy(x, BFLOAT16)
    got = ex.exec_transform_bool(TransformBool.MatchConditionBool, X, extra_args=[1.0, 0.0, mode]).to_numpy()
    assert np.array_equal(got, O.match_mask(x, 1.0, 0.0, mode))


@pytest.mark.parametrize("dt", FLOATS + [INT32])
@pytest.mark.parametrize("mode", [0, 1, 2, 5, 9, 10, 11, 13])
def test_compare_and_set_and_replace_pairwise_and_scalar(ex, dt, mode):
    rng = np.random.default_rng(300 + mode + 16 * dt)
    x, y = _draw(rng, (45, 77), dt), _draw(rng, (45, 77), dt)
    compare, eps = (1.0, 1.0) if dt in (INT32, INT64) else (1.0, 0.5)
    X, Y = NDArray.from_numpy(x), NDArray.from_numpy(y)
    params = [compare, 0.0, eps, mode]
    assert _same(ex.exec_pairwise(Pairwise.CompareAndSet, X, Y, extra_args=params).to_numpy(), O.compare_and_set(x, y, compare, eps, mode))
    assert _same(ex.exec_pairwise(Pairwise.CompareAndReplace, X, Y, extra_args=params).to_numpy(), O.compare_and_replace(x, y, compare, eps, mode))
    for s in (1.0, 3.0):
        want = O.compare_and_set(x, np.full(x.shape, s, NP[dt]), compare, eps, mode)
        assert _same(ex.exec_scalar(Scalar.CompareAndSet, X, s, extra_args=params).to_numpy(), want)


@pytest.mark.parametrize("dt", FLOATS + [INT32, INT64])
@pytest.mark.parametrize("mode", [0, 1, 2, 7, 8, 9, 10, 14])
def test_match_count_and_first_last_index(ex, dt, mode):
    rng = np.random.default_rng(500 + mode + 16 * dt)
    x = _draw(rng, (9, 14, 11), dt)
    x[3] = 3 if dt in (INT32, INT64) else 3.5              # a slab where most conditions have no hit at all, or only hits
    compare, eps = (1.0, 1.0) if dt in (INT32, INT64) else (1.0, 0.5)
    X = NDArray.from_numpy(x)
    params = [compare, eps, mode]
    for dims in (None, [2], [0], [1, 2], [0, 2]):
        want = O.match_count(x, compare, eps, mode, dims)
        got = ex.exec_reduce_long(ReduceLong.MatchCondition, X, dims, extra_args=params).to_numpy()
        assert np.array_equal(got.reshape(np.shape(want)), want), dims
        for op, last in ((IndexReduce.FirstIndex, False), (IndexReduce.LastIndex, True)):
            want = O.first_last_index(x, compare, eps, mode, dims, last=last)
            got = ex.exec_index_reduce(op, X, dims, extra_args=params).to_numpy()
            assert np.array_equal(got.reshape(np.shape(want)), want), (dims, last)


@pytest.mark.parametrize("dt", [FLOAT32, INT64])
def test_long_rows_split_over_blocks(ex, dt):
    """Rows long enough for the partial / finish pair: one hit, two hits, none."""
    n = 300_007
    x = np.zeros((3, n), NP[dt])
    x[0, 123_456] = 2
    x[1, 17] = 2; x[1, n - 5] = 2
    X = NDArray.from_numpy(x)
    params = [2.0, 0.0, 10]
    assert np.array_equal(ex.exec_reduce_long(ReduceLong.MatchCondition, X, [1], extra_args=params).to_numpy(), [1, 2, 0])
    assert np.array_equal(ex.exec_index_reduce(IndexReduce.FirstIndex, X, [1], extra_args=params).to_numpy(), [123_456, 17, -1])
    assert np.array_equal(ex.exec_index_reduce(IndexReduce.LastIndex, X, [1], extra_args=params).to_numpy(), [123_456, n - 5, -1])
    assert int(ex.exec_index_reduce(IndexReduce.FirstIndex, X, None, extra_args=params).to_numpy()) == 123_456
    assert int(ex.exec_index_reduce(IndexReduce.LastIndex, X, None, extra_args=params).to_numpy()) == 2 * n - 5
    assert int(ex.exec_reduce_long(ReduceLong.MatchCondition, X, None, extra_args=[0.0, 0.0, 11]).to_numpy()) == 3


def test_reference_held_vectors(ex):
    """The cases the reference's own tests state, through the HIP path."""
    x5 = NDArray.from_numpy(np.array([[1, 2, 3, 4, 5]], np.float64))
    assert int(ex.exec_index_reduce(IndexReduce.FirstIndex, x5, None, extra_args=[3.0, 0.0, 10.0]).to_numpy()) == 2   # NDArrayTests2.cpp:96-103
    x = np.array([1, 2, 0, 4, 5], np.float64)
    X = NDArray.from_numpy(x)
    comp = NDArray.from_numpy(np.array([1, 2, 3, 4, 5], np.float64))
    cst = lambda p: ex.exec_transform_same(TransformSame.CompareAndSetTransform, X, extra_args=p).to_numpy()
    assert np.array_equal(cst([0.0, 3.0, EPS, 0]), [1, 2, 3, 4, 5])
    assert np.array_equal(cst([2.0, 3.0, EPS, 2]), [3, 2, 3, 4, 5])
    assert np.array_equal(ex.exec_pairwise(Pairwise.CompareAndSet, X, comp, extra_args=[5.0, 0.0, EPS, 2]).to_numpy(), [1, 2, 3, 4, 5])
    assert np.array_equal(ex.exec_pairwise(Pairwise.CompareAndReplace, X, comp, extra_args=[1.0, 0.0, EPS, 2]).to_numpy(), [1, 2, 3, 4, 5])
    y = NDArray.from_numpy(np.array([2, 4, 3, 0, 5], np.float64))
    assert np.array_equal(ex.exec_pairwise(Pairwise.CompareAndSet, X, y, extra_args=[0.0, 0.0, EPS, 1]).to_numpy(), [2, 4, 3, 4, 5])
    y2 = NDArray.from_numpy(np.array([2, 4, 3, 4, 5], np.float64))
    car = lambda p: ex.exec_pairwise(Pairwise.CompareAndReplace, X, y2, extra_args=p).to_numpy()
    assert np.array_equal(car([0.0, 0.0, EPS, 1]), [2, 4, 0, 4, 5])
    assert np.array_equal(car([4.0, 0.0, EPS, 2]), [2, 4, 3, 4, 5])
    assert np.array_equal(car([2.0, 0.0, EPS, 2]), [2, 2, 3, 4, 5])
    a = np.arange(10, dtype=np.float64)
    cnt = lambda v, p: int(ex.exec_reduce_long(ReduceLong.MatchCondition, NDArray.from_numpy(v), None, extra_args=p).to_numpy())
    assert cnt(a, [5.0, EPS, 2]) == 5
    b = a.copy(); b[4] = np.nan
    assert cnt(b, [0.0, EPS, 9]) == 1
    c = a.copy(); c[4] = -np.inf
    assert cnt(c, [0.0, EPS, 8]) == 1
    m = np.ones((3, 10)); m[2] = 0
    got = ex.exec_reduce_long(ReduceLong.MatchCondition, NDArray.from_numpy(m), [1], extra_args=[0.0, EPS, 0]).to_numpy()
    assert np.array_equal(got, [0, 0, 10])


@pytest.mark.parametrize("dt,rtol", [(DOUBLE, 1e-12), (FLOAT32, 2e-6), (HALF, 2e-3)])
@pytest.mark.parametrize("p", [1.0, 2.0, 3.0, 0.5])
def test_norm_p(ex, dt, rtol, p):
    rng = np.random.default_rng(int(p * 10) + dt)
    x = rng.standard_normal((12, 17, 9)).astype(NP[dt])
    X = NDArray.from_numpy(x)
    for dims in (None, [2], [0, 1], [1]):
        with np.errstate(over="ignore"):
            want = O.norm_p(x, p, dims).astype(NP[dt]).astype(np.float64)   # a HALF result past 65504 is inf on both sides
        got = ex.exec_reduce_float(ReduceFloat.NormP, X, dims, extra_args=[p]).to_numpy().astype(np.float64)
        np.testing.assert_allclose(got.reshape(np.shape(want)), want, rtol=rtol)
    # closed forms
    v = NDArray.from_numpy(np.array([3.0, -4.0], NP[dt]))
    assert float(ex.exec_reduce_float(ReduceFloat.NormP, v, None, extra_args=[2.0]).to_numpy()) == 5.0
    assert float(ex.exec_reduce_float(ReduceFloat.NormP, v, None, extra_args=[1.0]).to_numpy()) == 7.0


@pytest.mark.parametrize("dt", [DOUBLE, FLOAT32])
def test_equals_with_eps(ex, dt):
    rng = np.random.default_rng(dt)
    x = rng.standard_normal((6, 50)).astype(NP[dt])
    y = x.copy()
    y[1, 7] += 1e-3           # one pair outside the tolerance
    y[4] += 1e-7 if dt == DOUBLE else 0.0
    X, Y = NDArray.from_numpy(x), NDArray.from_numpy(y)
    params = [0.0, 0.0, 1e-5]
    got = ex.exec_reduce3(Reduce3.EqualsWithEps, X, Y, [1], extra_args=params).to_numpy()
    assert np.array_equal(got, O.equals_with_eps(x, y, 1e-5, [1]))
    assert np.array_equal(got, [1, 0, 1, 1, 1, 1])
    assert float(ex.exec_reduce3(Reduce3.EqualsWithEps, X, Y, None, extra_args=params).to_numpy()) == 0.0
    assert float(ex.exec_reduce3(Reduce3.EqualsWithEps, X, X, None, extra_args=params).to_numpy()) == 1.0
    assert float(ex.exec_reduce3(Reduce3.EqualsWithEps, X, Y, None, extra_args=[0.0, 0.0, 1e-2]).to_numpy()) == 1.0


def test_int64_values_are_refused(ex):
    """The value-carrying ops pass values through a double; INT64 arrays are an error rather than silently rounded."""
    from deeplearning4j_amd.nativeops import NativeOpsError
    X = NDArray.from_numpy(np.arange(8, dtype=np.int64))
    with pytest.raises(NativeOpsError):
        ex.exec_transform_same(TransformSame.CompareAndSetTransform, X, extra_args=[1.0, 2.0, 0.0, 10])
    with pytest.raises(NativeOpsError):
        ex.exec_pairwise(Pairwise.CompareAndSet, X, X, extra_args=[1.0, 0.0, 0.0, 10])
    with pytest.raises(NativeOpsError):
        ex.exec_scalar(Scalar.CompareAndSet, X, 3, extra_args=[1.0, 0.0, 0.0, 10])


def test_missing_extra_params_is_an_error(ex):
    from deeplearning4j_amd.nativeops import NativeOpsError
    X = NDArray.from_numpy(np.ones(8, np.float32))
    with pytest.raises(NativeOpsError):
        ex.exec_transform_bool(TransformBool.MatchConditionBool, X)
    with pytest.raises(NativeOpsError):
        ex.exec_reduce_float(ReduceFloat.NormP, X, None)
    with pytest.raises(NativeOpsError):
        ex.exec_index_reduce(IndexReduce.FirstIndex, X, None)
