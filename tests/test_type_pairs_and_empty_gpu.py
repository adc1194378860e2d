"""GPU parity of the operand-type pairs and EMPTY-array rules of the legacy loops, through the C ABI against the CPU oracle:
ReduceFloat of any numeric X into any float Z (NativeOpExecutioner_reduce.cpp:34-37,104-106), TransformFloat of integer and
bool X (NativeOpExecutioner_transform.cpp:35-37), reductions of EMPTY arrays (reduce_same.hpp:47,166-176,
reduce_float.hpp:243-251, ...), the transforms whose reference macros return their input or a constant, matmul of integer
arrays (MmulHelper.cpp:35-110).  Gates: fp32 results |a-b| <= 1e-6 + 1e-5 |b| (reductions: the absolute term scaled by
sum |x| eps), fp64 1e-12, 16-bit 1e-2; integer and bool results and fills must be equal."""
import numpy as np
import pytest

from conftest import assert_close
from deeplearning4j_amd import nativeops as N
from deeplearning4j_amd.executioner import (IndexReduce, ReduceBool, ReduceFloat, ReduceLong, ReduceSame, Reduce3, TransformFloat, TransformSame,
                                            TransformStrict)
from deeplearning4j_amd.ndarray import BFLOAT16, BOOL, DOUBLE, FLOAT32, HALF, INT32, INT64, NDArray, bf16_bits_to_f32, f32_to_bf16_bits

pytestmark = pytest.mark.gpu

NP = {FLOAT32: np.float32, DOUBLE: np.float64, HALF: np.float16, INT32: np.int32, INT64: np.int64, BOOL: np.bool_}
ZTOL = {FLOAT32: (1e-5, 1e-6), DOUBLE: (1e-12, 1e-12), HALF: (1e-2, 1e-3), BFLOAT16: (1e-2, 1e-3)}


def _input(rng, shape, dt):
    """(oracle array, device array, values as float64)"""
    from oracle import oracle as O
    if dt == BOOL:
        a = rng.integers(0, 2, shape).astype(np.bool_)
    elif dt in (INT32, INT64):
        a = rng.integers(-40, 41, shape).astype(NP[dt])
    elif dt == BFLOAT16:
        bits = f32_to_bf16_bits(rng.uniform(0.05, 0.95, shape).astype(np.float32))
        return O.Arr(bits, O.BFLOAT16), NDArray.from_numpy(bits, BFLOAT16), bf16_bits_to_f32(bits).astype(np.float64)
    else:
        a = rng.uniform(0.05, 0.95, shape).astype(NP[dt])
    return O.Arr(a), NDArray.from_numpy(a), a.astype(np.float64)


def _zero(oracle, shape, dt):
    if dt == BFLOAT16:
        return oracle.Arr(np.zeros(shape, np.uint16), oracle.BFLOAT16)
    return oracle.Arr(np.zeros(shape, NP[dt]))


def _close(got, want, rtol, atol, what):
    """assert_close, with equal infinities and NaN on both sides counting as equal (a HALF result may overflow on both sides)"""
    got, want = np.array(got, np.float64), np.array(want, np.float64)
    same = (got == want) | (np.isnan(got) & np.isnan(want))
    assert_close(np.where(same, 0.0, got), np.where(same, 0.0, want), rtol, atol, what)


def _values(a, dt):
    return bf16_bits_to_f32(a).astype(np.float64) if dt == BFLOAT16 else np.asarray(a, np.float64)


def test_reference_vectors_mean_of_an_integer_array(ex):
    # MultiDataTypeTests.cpp:246-256 (ndarray_reduceAlongDimension_test2): Mean of INT32 {0, 1, 2, 3} -> FLOAT32 1.5, [0.5, 2.5]
    x = NDArray.from_numpy(np.array([[0, 1], [2, 3]], np.int32))
    assert ex.exec_reduce_float(ReduceFloat.Mean, x).to_numpy() == np.float32(1.5)
    got = ex.exec_reduce_float(ReduceFloat.Mean, x, [1])
    assert got.dtype == FLOAT32 and np.array_equal(got.to_numpy(), np.array([0.5, 2.5], np.float32))


@pytest.mark.parametrize("zdt", [FLOAT32, DOUBLE, HALF, BFLOAT16])
@pytest.mark.parametrize("xdt", [FLOAT32, DOUBLE, HALF, BFLOAT16, INT32, INT64, BOOL])
def test_reduce_float_every_input_type_into_every_float_type(ex, oracle, xdt, zdt):
    rng = np.random.default_rng(1000 + 20 * xdt + zdt)
    shape = (23, 301)
    ox, X, vals = _input(rng, shape, xdt)
    ops = [ReduceFloat.Mean, ReduceFloat.AMean, ReduceFloat.Norm1, ReduceFloat.Norm2, ReduceFloat.NormMax, ReduceFloat.SquaredNorm]
    if xdt not in (INT32, INT64, BOOL):
        ops += [ReduceFloat.Entropy, ReduceFloat.LogEntropy, ReduceFloat.ShannonEntropy]      # x log x needs positive inputs
    rtol, atol = ZTOL[zdt]
    scale = np.abs(vals).sum(1).max() * (2.0 ** -23 if zdt != DOUBLE else 2.0 ** -52) * 8
    for op in ops:
        for dims, zshape in (([1], (23,)), (None, ())):
            want = oracle.reduce_float(op, ox, _zero(oracle, zshape, zdt), dims)
            got = ex.exec_reduce_float(op, X, dims, z=NDArray.empty(zshape, zdt)).to_numpy()
            big = scale * (np.abs(vals).max() + 1.0) * (vals.shape[0] if dims is None else 1)
            # the entropies take the logarithm in X's type: two float logarithm routines may differ in the last place, which a
            # 16-bit X can turn into one unit of ITS last place in a term or two of a row
            r = rtol
            if op in (ReduceFloat.Entropy, ReduceFloat.LogEntropy, ReduceFloat.ShannonEntropy) and xdt != DOUBLE:
                r = max(rtol, 1e-4 if xdt in (HALF, BFLOAT16) else 1e-6)
            _close(_values(got, zdt), _values(want, zdt), r, atol + big, "op %d dims %s" % (op, dims))
    # a long run split over several blocks, and a strided view
    ox2, X2, v2 = _input(rng, (3, 70001), xdt)
    want = oracle.reduce_float(ReduceFloat.Mean, ox2, _zero(oracle, (3,), zdt), [1])
    got = ex.exec_reduce_float(ReduceFloat.Mean, X2, [1], z=NDArray.empty((3,), zdt)).to_numpy()
    _close(_values(got, zdt), _values(want, zdt), rtol, atol + 1e-4, "long rows")
    want = oracle.reduce_float(ReduceFloat.Norm1, oracle.Arr(ox.a.T, ox.dt), _zero(oracle, (301,), zdt), [1])
    got = ex.exec_reduce_float(ReduceFloat.Norm1, X.permute(1, 0), [1], z=NDArray.empty((301,), zdt)).to_numpy()
    _close(_values(got, zdt), _values(want, zdt), rtol, atol + scale * 50, "transposed view")


@pytest.mark.parametrize("zdt", [FLOAT32, DOUBLE, HALF, BFLOAT16])
@pytest.mark.parametrize("xdt", [INT32, INT64, BOOL])
def test_transform_float_of_integer_and_bool_arrays(ex, oracle, xdt, zdt):
    rng = np.random.default_rng(xdt * 7 + zdt)
    a = rng.integers(0, 2, (17, 33)).astype(np.bool_) if xdt == BOOL else rng.integers(1, 5000, (17, 33)).astype(NP[xdt])
    X = NDArray.from_numpy(a)
    rtol, atol = ZTOL[zdt]
    for op in (TransformFloat.Sqrt, TransformFloat.RSqrt):
        if op == TransformFloat.RSqrt and xdt == BOOL:
            continue                                          # 1 / sqrt(0)
        want = oracle.transform_float(op, a, _zero(oracle, a.shape, zdt))
        got = ex.exec_transform_float(op, X, z=NDArray.empty(a.shape, zdt)).to_numpy()
        assert_close(_values(got, zdt), _values(want, zdt), rtol, atol, "op %d" % op)
        # a transposed view into a dense result
        want = oracle.transform_float(op, np.ascontiguousarray(a.T), _zero(oracle, a.T.shape, zdt))
        got = ex.exec_transform_float(op, X.permute(1, 0), z=NDArray.empty(a.T.shape, zdt)).to_numpy()
        assert_close(_values(got, zdt), _values(want, zdt), rtol, atol, "view, op %d" % op)
    assert ex.exec_transform_float(TransformFloat.Sqrt, X).dtype == FLOAT32     # the default result type


def test_reference_vectors_reductions_of_empty_arrays(ex):
    # LegacyOpsTests.cpp:616-658 (test_legacy_reduce_empty_1/2/3): x [2, 0, 3] reduced along 1 into [2, 3]
    x = NDArray.empty((2, 0, 3), FLOAT32)
    z = NDArray.from_numpy(np.full((2, 3), 7.0, np.float32))
    assert np.array_equal(ex.exec_reduce_same(ReduceSame.Sum, x, [1], z=z).to_numpy(), np.zeros((2, 3), np.float32))
    assert np.array_equal(ex.exec_reduce_same(ReduceSame.Min, x, [1], z=z).to_numpy(), np.full((2, 3), np.inf, np.float32))
    assert np.array_equal(ex.exec_reduce_same(ReduceSame.Max, x, [1], z=z).to_numpy(), np.full((2, 3), -np.inf, np.float32))
    # :660-676 (test_legacy_reduce_empty_4): an EMPTY result is left alone
    ex.exec_reduce_same(ReduceSame.Sum, NDArray.empty((1, 0, 2), FLOAT32), [0], z=NDArray.empty((0, 2), FLOAT32))
    # DeclarableOpsTests14.cpp:230-265: reduce_min / reduce_sum / reduce_mean of a float [1, 0] along 1, keepDims
    e = NDArray.empty((1, 0), FLOAT32)
    assert ex.exec_custom("reduce_min", [e], t_args=[1.0], i_args=[1])[0].to_numpy().reshape(-1)[0] == np.inf
    assert ex.exec_custom("reduce_sum", [e], t_args=[1.0], i_args=[1])[0].to_numpy().reshape(-1)[0] == 0.0
    assert np.isnan(ex.exec_custom("reduce_mean", [e], t_args=[1.0], i_args=[1])[0].to_numpy().reshape(-1)[0])
    # LegacyOpsTests.cpp:678-690 (test_legacy_transform_float_1): a float transform of an EMPTY array does nothing
    t = NDArray.empty((1, 0, 4), FLOAT32)
    ex.exec_transform_float(TransformFloat.RSqrt, t, z=t)


@pytest.mark.parametrize("dt", [FLOAT32, DOUBLE, HALF, BFLOAT16, INT32, INT64])
def test_reductions_of_empty_arrays_fill_the_starting_value(ex, oracle, dt):
    name = {FLOAT32: np.dtype(np.float32), DOUBLE: np.dtype(np.float64), HALF: "float16", BFLOAT16: "bfloat16", INT32: np.dtype(np.int32), INT64: np.dtype(np.int64)}
    x = NDArray.empty((4, 0, 5), dt)
    def filled(z, want, what):
        got = _values(z.to_numpy(), z.dtype)
        if isinstance(want, float) and np.isnan(want):
            assert np.isnan(got).all(), what
        else:
            assert np.array_equal(got, np.full(got.shape, float(want))), (what, got, want)
    for op in (ReduceSame.Sum, ReduceSame.Max, ReduceSame.Min, ReduceSame.Prod, ReduceSame.ASum):
        want = oracle.reduce_of_empty("same", op, name[dt], name[dt])
        filled(ex.exec_reduce_same(op, x, [1]), want, ("same along a dim", op))
        filled(ex.exec_reduce_same(op, x), want, ("same, whole array", op))
    with pytest.raises(N.NativeOpsError, match="first element"):
        ex.exec_reduce_same(ReduceSame.AMax, x)
    for zdt in (FLOAT32, DOUBLE, HALF, BFLOAT16):
        for op in (ReduceFloat.Mean, ReduceFloat.AMean, ReduceFloat.Norm2, ReduceFloat.NormMax, ReduceFloat.Entropy):
            want = oracle.reduce_of_empty("float", op, name[dt], name[zdt])
            filled(ex.exec_reduce_float(op, x, [1], z=NDArray.from_numpy(np.ones((4, 5), np.float32), zdt) if zdt == BFLOAT16 else NDArray.from_numpy(np.ones((4, 5), NP[zdt]))), want, ("float", op, zdt))
        filled(ex.exec_reduce_float(ReduceFloat.NormP, x, z=NDArray.scalar(3.0, zdt), extra_args=[2.0]), 0.0, ("NormP", zdt))
    for op in (IndexReduce.IndexMax, IndexReduce.IndexMin, IndexReduce.IndexAbsoluteMax):
        filled(ex.exec_index_reduce(op, x, [1], z=NDArray.from_numpy(np.full((4, 5), 9, np.int64))), 0, ("index", op))
    filled(ex.exec_index_reduce(IndexReduce.FirstIndex, x, [1], z=NDArray.from_numpy(np.full((4, 5), 9, np.int64)), extra_args=[1.0, 0.0, 2.0]), -1, "FirstIndex")
    filled(ex.exec_reduce_long(ReduceLong.CountNonZero, x, [1], z=NDArray.from_numpy(np.full((4, 5), 9, np.int64))), 0, "CountNonZero")
    filled(ex.exec_reduce_long(ReduceLong.MatchCondition, x, [1], z=NDArray.from_numpy(np.full((4, 5), 9, np.int64)), extra_args=[1.0, 0.0, 2.0]), 0, "MatchCondition")
    filled(ex.exec_reduce_bool(ReduceBool.All, x), 1, "All")
    filled(ex.exec_reduce_bool(ReduceBool.Any, x), 0, "Any")
    filled(ex.exec_reduce_bool(ReduceBool.IsNan, x), 0, "IsNan")
    # reduce3 with an EMPTY operand writes nothing (loops/cpu/reduce3.hpp:49-57: its fill loop runs over x's zero elements)
    if dt in (FLOAT32, DOUBLE):
        z = NDArray.from_numpy(np.full((4, 5), 3.0, NP[dt]))
        ex.exec_reduce3(Reduce3.Dot, x, x, [1], z=z)
        assert np.array_equal(z.to_numpy(), np.full((4, 5), 3.0, NP[dt]))


@pytest.mark.parametrize("dt", [FLOAT32, DOUBLE, HALF, BFLOAT16])
def test_transforms_whose_reference_macros_return_the_input_or_a_constant(ex, oracle, dt):
    v = np.array([-3.0, -2.5, -1.0, -0.5, -0.0, 0.0, 0.5, 1.0, 2.5, 2.625, 7.0, np.nan, np.inf, -np.inf] * 5)
    if dt == BFLOAT16:
        bits = f32_to_bf16_bits(v.astype(np.float32))
        ox, X = oracle.Arr(bits, oracle.BFLOAT16), NDArray.from_numpy(bits, BFLOAT16)
    else:
        ox, X = oracle.Arr(v.astype(NP[dt])), NDArray.from_numpy(v.astype(NP[dt]))
    for op in (TransformStrict.HardTanhDerivative, TransformStrict.HardSigmoidDerivative, TransformStrict.StabilizeFP16):
        want = oracle.transform_strict(op, ox, _zero(oracle, v.shape, dt))
        got = ex.exec_transform_strict(op, X).to_numpy()
        assert np.array_equal(_values(got, dt), _values(want, dt), equal_nan=True), op
    want = oracle.transform_same(TransformSame.Sign, ox, _zero(oracle, v.shape, dt))
    got = ex.exec_transform_same(TransformSame.Sign, X).to_numpy()
    assert np.array_equal(_values(got, dt), _values(want, dt)), "Sign"
    assert _values(got, dt)[0] == 1.0 and _values(got, dt)[4] == -1.0 and _values(got, dt)[11] == -1.0   # -3 -> 1, -0 -> -1, NaN -> -1


@pytest.mark.parametrize("dt", [INT32, INT64])
def test_sign_of_integer_arrays(ex, dt):
    a = np.array([-5, -1, 0, 1, 9, 0, -2 ** 31 + 1], NP[dt])
    assert np.array_equal(ex.exec_transform_same(TransformSame.Sign, NDArray.from_numpy(a)).to_numpy(), np.where(a != 0, 1, -1).astype(NP[dt]))


@pytest.mark.parametrize("dt", [INT32, INT64])
def test_matmul_of_integer_arrays(ex, oracle, dt):
    rng = np.random.default_rng(dt)
    # DeclarableOpsTests-style exact case, then random operands large enough to wrap around
    got = ex.exec_custom("matmul", [NDArray.from_numpy(np.array([[1, 2], [3, 4]], NP[dt])), NDArray.from_numpy(np.array([[5, 6], [7, 8]], NP[dt]))])[0]
    assert got.dtype == dt and np.array_equal(got.to_numpy(), [[19, 22], [43, 50]])
    bits = 32 if dt == INT32 else 64
    for (m, k, n) in ((7, 13, 5), (64, 300, 33), (1, 17, 9), (130, 1, 4)):
        a = rng.integers(-2 ** (bits - 3), 2 ** (bits - 3), (m, k)).astype(NP[dt])
        b = rng.integers(-2 ** (bits - 3), 2 ** (bits - 3), (k, n)).astype(NP[dt])
        assert np.array_equal(ex.exec_custom("matmul", [NDArray.from_numpy(a), NDArray.from_numpy(b)])[0].to_numpy(), oracle.matmul_int(a, b)), (m, k, n)
        # transposed operands are strides, alpha and beta are cast to the arrays' type (2.9 -> 2)
        c = rng.integers(-50, 50, (m, n)).astype(NP[dt])
        C = NDArray.from_numpy(c)
        ex.exec_custom("matmul", [NDArray.from_numpy(np.ascontiguousarray(a.T)), NDArray.from_numpy(np.ascontiguousarray(b.T))], outputs=[C], t_args=[2.9, 3.0], i_args=[1, 1, 0])
        assert np.array_equal(C.to_numpy(), oracle.matmul_int(a, b, c, 2.9, 3.0)), ("flags", m, k, n)
    # batched
    a = rng.integers(-1000, 1000, (3, 4, 6)).astype(NP[dt]); b = rng.integers(-1000, 1000, (3, 6, 5)).astype(NP[dt])
    assert np.array_equal(ex.exec_custom("matmul", [NDArray.from_numpy(a), NDArray.from_numpy(b)])[0].to_numpy(), oracle.matmul_int(a, b))
    assert N.load().nd4jhipLastGemmKernel().decode().startswith("gemm_int")
