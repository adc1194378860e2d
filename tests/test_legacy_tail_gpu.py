"""GPU parity of the rest of the legacy op tables (transform strict/same, pairwise, scalar, broadcast): every opNum
the library accepts beyond the hot ones runs through the C ABI and is compared with the CPU oracle on the same
inputs.  Gates: fp32 |a-b| <= 1e-6 + 1e-5 |b|; fp64 1e-12 relative (1e-9 where the two sides use different
exp/pow routines); fp16/bf16 1e-2.  Integer-valued results (rounding, logical, truncating ops) must be equal.
"""
import numpy as np
import pytest

from conftest import assert_close
from deeplearning4j_amd.executioner import Broadcast, Pairwise, ReduceFloat, Scalar, TransformSame, TransformStrict
from deeplearning4j_amd.ndarray import BFLOAT16, DOUBLE, FLOAT32, HALF, NDArray, bf16_bits_to_f32, f32_to_bf16_bits

pytestmark = pytest.mark.gpu

TS = TransformStrict
STRICT_TAIL = [TS.TanhDerivative, TS.SigmoidDerivative, TS.SoftSignDerivative, TS.TanDerivative, TS.SELUDerivative,
               TS.RationalTanhDerivative, TS.RectifiedTanhDerivative, TS.SwishDerivative, TS.ACoshDerivative, TS.ASinhDerivative,
               TS.SinhDerivative, TS.LogSigmoidDerivative, TS.SpecialDerivative, TS.CubeDerivative, TS.ACos, TS.ASin, TS.ATan,
               TS.HardTanh, TS.SoftSign, TS.HardSigmoid, TS.RationalTanh, TS.RectifiedTanh, TS.Sinh, TS.Cosh, TS.Tan, TS.SELU,
               TS.Log1p, TS.ACosh, TS.ASinh, TS.Rint, TS.LogSigmoid, TS.Erfc, TS.Expm1, TS.ATanh, TS.GELUDerivative,
               TS.PreciseGELUDerivative, TS.Mish, TS.MishDerivative]
TOL = {FLOAT32: (1e-5, 1e-6), DOUBLE: (1e-9, 1e-12), HALF: (1e-2, 1e-3), BFLOAT16: (1e-2, 1e-3)}


def _pair(oracle, a, dtype):
    if dtype == BFLOAT16:
        bits = f32_to_bf16_bits(a.astype(np.float32))
        return oracle.Arr(bits, oracle.BFLOAT16), NDArray.from_numpy(bits, BFLOAT16)
    np_dt = {HALF: np.float16, DOUBLE: np.float64, FLOAT32: np.float32}[dtype]
    v = a.astype(np_dt)
    return oracle.Arr(v), NDArray.from_numpy(v)


def _zeros(oracle, oa, shape=None):
    return oracle.Arr(np.zeros(shape or oa.a.shape, oa.a.dtype), oa.dt)


def _f(oa):
    return bf16_bits_to_f32(oa.a) if oa.dt == 17 else oa.a.astype(np.float64)


def _got(nd, dtype):
    return nd.to_numpy() if dtype == DOUBLE else nd.to_float()


def _domain(op, rng, shape):
    a = rng.uniform(-3, 3, shape)
    if op in (TS.ACos, TS.ASin, TS.ATanh):
        a = rng.uniform(-0.9, 0.9, shape)
    elif op in (TS.ACosh, TS.ACoshDerivative):
        a = rng.uniform(1.25, 6, shape)
    elif op == TS.Log1p:
        a = rng.uniform(-0.75, 5, shape)
    elif op in (TS.Tan, TS.TanDerivative):
        a = rng.uniform(-1.3, 1.3, shape)
    elif op == TS.Rint:
        a = np.round(rng.uniform(-6, 6, shape) * 4) / 4          # quarters: exact halves occur
    return a


@pytest.mark.parametrize("op", STRICT_TAIL)
@pytest.mark.parametrize("dtype", [FLOAT32, BFLOAT16, HALF, DOUBLE])
def test_transform_strict_tail(ex, oracle, op, dtype):
    rng = np.random.default_rng(900 + op)
    a = _domain(op, rng, (67, 131))
    ox, dx = _pair(oracle, a, dtype)
    oz = _zeros(oracle, ox)
    oracle.transform_strict(op, ox, oz)
    got = ex.exec_transform_strict(op, dx)
    rtol, atol = TOL[dtype]
    if op in (TS.Rint, TS.HardTanh) or (op == TS.RectifiedTanhDerivative and False):
        assert np.array_equal(_got(got, dtype), _f(oz)), "op %d dtype %d" % (op, dtype)
    else:
        assert_close(_got(got, dtype), _f(oz), rtol, atol, "strict tail op %d dtype %d" % (op, dtype))


def test_transform_strict_tail_on_a_permuted_view_and_odd_length(ex, oracle):
    rng = np.random.default_rng(31)
    a = rng.uniform(-2, 2, (6, 10, 14)).astype(np.float32)
    A = NDArray.from_numpy(a)
    got = ex.exec_transform_strict(TS.Mish, A.permute(2, 0, 1), NDArray.empty((14, 6, 10), FLOAT32))
    want = oracle.transform_strict(TS.Mish, a.transpose(2, 0, 1), np.zeros((14, 6, 10), np.float32))
    assert_close(got.to_numpy(), want, 1e-5, 1e-6, "mish on a permuted view")
    b = rng.uniform(-2, 2, 1003).astype(np.float32)              # not a multiple of the vector width
    got = ex.exec_transform_strict(TS.SELU, NDArray.from_numpy(b))
    assert_close(got.to_numpy(), oracle.transform_strict(TS.SELU, b, np.zeros_like(b)), 1e-5, 1e-6, "selu, ragged length")


@pytest.mark.parametrize("dtype", [FLOAT32, BFLOAT16, HALF, DOUBLE])
def test_transform_same_tail(ex, oracle, dtype):
    rng = np.random.default_rng(41)
    a = np.round(rng.uniform(-5, 5, (33, 47)) * 8) / 8           # eighths: exact in every type, halves occur
    ox, dx = _pair(oracle, a, dtype)
    for op in (TransformSame.Ones, TransformSame.Round, TransformSame.TimesOneMinus, TransformSame.Ceiling, TransformSame.Floor):
        oz = _zeros(oracle, ox)
        oracle.transform_same(op, ox, oz)
        got = ex.exec_transform_same(op, dx)
        if op == TransformSame.TimesOneMinus and dtype in (HALF, BFLOAT16):
            assert_close(_got(got, dtype), _f(oz), 1e-2, 1e-3, "same op %d" % op)
        else:
            assert np.array_equal(_got(got, dtype), _f(oz)), "same op %d dtype %d" % (op, dtype)


def test_transform_same_rejects_unknown_op_numbers(ex):
    from deeplearning4j_amd.nativeops import NativeOpsError
    with pytest.raises(NativeOpsError, match="not implemented"):
        ex.exec_transform_same(9, NDArray.from_numpy(np.ones(4, np.float32)))


P = Pairwise
PAIRWISE_TAIL = [P.Pow, P.Copy2, P.Remainder, P.FMod, P.Atan2, P.TruncateDiv, P.FloorDiv, P.FloorMod, P.ReverseMod, P.SafeDivide, P.Mod,
                 P.LogicalOr, P.LogicalXor, P.LogicalNot, P.LogicalAnd, P.AMaxPairwise, P.AMinPairwise, P.TruncateMod, P.ReplaceNans,
                 P.DivideNoNan]
EXACT_BINARY = {"TruncateDiv", "FloorDiv", "ReverseMod", "LogicalOr", "LogicalXor", "LogicalNot", "LogicalAnd", "AMaxPairwise",
                "AMinPairwise", "TruncateMod", "ReplaceNans", "Copy2", "CopyPws", "MaxPairwise", "MinPairwise", "Step", "RELU", "RELU6",
                "RELUDerivative", "LstmClip", "LeakyRELUDerivative"}


def _binary_inputs(rng, shape, name):
    # quarters keep remainders exact in bf16/half; divisors stay >= 1 in magnitude so (int) casts are non-zero
    a = np.round(rng.uniform(-8, 8, shape) * 4) / 4
    b = np.round(rng.uniform(1, 5, shape) * 4) / 4 * rng.choice([-1.0, 1.0], shape)
    if name in ("Pow", "ReversePow", "LogX"):
        a = np.abs(a) + 0.5
        b = np.abs(b)
    if name == "ReverseMod":
        a = np.where(np.abs(a) < 1, 2.0, a)
    if name == "ReplaceNans":
        a = np.where(rng.uniform(size=shape) < 0.2, np.nan, a)
    if name in ("SafeDivide", "DivideNoNan"):
        b = np.where(rng.uniform(size=shape) < 0.2, 0.0, b)
    return a, b


def _name(cls, op):
    return [k for k, v in vars(cls).items() if v == op and not k.startswith("_")][0]


def _check_binary(name, got, want, dtype, what):
    if name in EXACT_BINARY:
        assert np.array_equal(got, want, equal_nan=True), what
    else:
        rtol, atol = TOL[dtype]
        assert_close(got, want, rtol, atol, what)


@pytest.mark.parametrize("op", PAIRWISE_TAIL)
@pytest.mark.parametrize("dtype", [FLOAT32, BFLOAT16, HALF, DOUBLE])
def test_pairwise_tail(ex, oracle, op, dtype):
    name = _name(Pairwise, op)
    rng = np.random.default_rng(700 + op)
    a, b = _binary_inputs(rng, (37, 53), name)
    if name == "Pow" and dtype in (HALF, BFLOAT16):
        b = np.minimum(b, 3.0)
    ox, dx = _pair(oracle, a, dtype)
    oy, dy = _pair(oracle, b, dtype)
    oz = _zeros(oracle, ox)
    oracle.pairwise(op, ox, oy, oz)
    got = ex.exec_pairwise(op, dx, dy)
    _check_binary(name, _got(got, dtype), _f(oz), dtype, "pairwise %s dtype %d" % (name, dtype))


def test_pairwise_tail_strided_operands(ex, oracle):
    rng = np.random.default_rng(77)
    a = np.round(rng.uniform(-8, 8, (12, 20)) * 4).astype(np.float32) / 4
    b = (np.round(rng.uniform(1, 5, (20, 12)) * 4) / 4).astype(np.float32)
    A, B = NDArray.from_numpy(a), NDArray.from_numpy(b)
    got = ex.exec_pairwise(P.FloorMod, A, B.permute(1, 0), NDArray.empty((12, 20), FLOAT32))
    want = oracle.pairwise(P.FloorMod, a, b.T, np.zeros((12, 20), np.float32))
    assert np.array_equal(got.to_numpy(), want)


S = Scalar
SCALAR_TAIL = [(S.ELU, 1.5), (S.ELUDerivative, 1.5), (S.Mod, 3.0), (S.ReverseMod, 7.0), (S.Remainder, 3.0), (S.FMod, 3.0), (S.TruncateDiv, 2.0),
               (S.FloorDiv, 2.0), (S.FloorMod, -3.0), (S.SquaredSubtract, 1.25), (S.SafeDivide, 0.0), (S.AMaxPairwise, 1.0),
               (S.AMinPairwise, 1.0), (S.Atan2, 2.0), (S.LogicalOr, 2.0), (S.LogicalXor, 3.0), (S.LogicalNot, 1.0), (S.LogicalAnd, 6.0),
               (S.Pow, 3.0), (S.SXELogitsSmoother, 0.125), (S.LeakyRELU, 0.125), (S.LeakyRELUDerivative, 0.125), (S.ReplaceNans, 4.0),
               (S.LogX, 2.0), (S.RELU, 0.0), (S.RELU6, 0.0), (S.Step, 0.25), (S.LstmClip, 2.0), (S.TruncateMod, 3.0),
               (S.SquaredReverseSubtract, 1.25), (S.ReversePow, 2.0), (S.DivideNoNan, 0.0), (S.RELUDerivative, 0.25)]


@pytest.mark.parametrize("op,value", SCALAR_TAIL)
@pytest.mark.parametrize("dtype", [FLOAT32, BFLOAT16, DOUBLE])
def test_scalar_tail(ex, oracle, op, value, dtype):
    name = _name(Scalar, op)
    rng = np.random.default_rng(500 + op)
    a, _ = _binary_inputs(rng, (29, 41), name)
    if name == "Pow" and dtype == BFLOAT16:
        a = np.clip(a, -4, 4)
    ox, dx = _pair(oracle, a, dtype)
    oz = _zeros(oracle, ox)
    oracle.scalar(op, ox, value, oz)
    got = ex.exec_scalar(op, dx, value)
    _check_binary(name, _got(got, dtype), _f(oz), dtype, "scalar %s dtype %d" % (name, dtype))


def test_scalar_tail_on_a_view(ex, oracle):
    rng = np.random.default_rng(78)
    a = rng.uniform(-3, 3, (8, 6, 10)).astype(np.float32)
    got = ex.exec_scalar(S.LeakyRELU, NDArray.from_numpy(a).permute(1, 2, 0), 0.01, NDArray.empty((6, 10, 8), FLOAT32))
    want = oracle.scalar(S.LeakyRELU, a.transpose(1, 2, 0), 0.01, np.zeros((6, 10, 8), np.float32))
    assert np.array_equal(got.to_numpy(), want)


B = Broadcast
BROADCAST_TAIL = [B.Pow, B.AMinPairwise, B.AMaxPairwise, B.FloorMod, B.FloorDiv, B.ReverseMod, B.SafeDivide, B.Mod, B.TruncateDiv, B.Atan2,
                  B.LogicalOr, B.LogicalXor, B.LogicalNot, B.LogicalAnd, B.DivideNoNan, B.MinPairwise, B.MaxPairwise, B.SquaredSubtract]


@pytest.mark.parametrize("op", BROADCAST_TAIL)
@pytest.mark.parametrize("dims", [[1], [0, 2]])
def test_broadcast_tail(ex, oracle, op, dims):
    name = _name(Broadcast, op)
    rng = np.random.default_rng(300 + op)
    shape = (5, 12, 7)
    a, _ = _binary_inputs(rng, shape, name)
    _, b = _binary_inputs(rng, tuple(shape[d] for d in dims), name)
    a, b = a.astype(np.float32), b.astype(np.float32)
    want = oracle.broadcast(op, a, b, np.zeros(shape, np.float32), dims)
    got = ex.exec_broadcast(op, NDArray.from_numpy(a), NDArray.from_numpy(b), dims)
    _check_binary(name, got.to_numpy().astype(np.float64), want.astype(np.float64), FLOAT32, "broadcast %s dims %s" % (name, dims))


@pytest.mark.parametrize("op", [ReduceFloat.Entropy, ReduceFloat.LogEntropy, ReduceFloat.ShannonEntropy])
@pytest.mark.parametrize("dtype", [FLOAT32, DOUBLE, BFLOAT16, HALF])
@pytest.mark.parametrize("dims", [[1], [0], None])
def test_entropy_reductions(ex, oracle, op, dtype, dims):
    rng = np.random.default_rng(60 + op)
    p = rng.uniform(0.05, 1, (48, 200))
    p /= p.sum(1, keepdims=True) if dims != [0] else p.sum(0, keepdims=True)
    if dims is None:
        p /= p.sum()
        p *= 4                        # keeps half-precision terms away from the subnormal range
    ox, dx = _pair(oracle, p, dtype)
    out_shape = () if dims is None else tuple(s for i, s in enumerate(p.shape) if i not in dims)
    oz = oracle.Arr(np.zeros(out_shape, ox.a.dtype), ox.dt)
    oracle.reduce_float(op, ox, oz, dims)
    got = ex.exec_reduce_float(op, dx, dims)
    rtol, atol = {FLOAT32: (2e-5, 1e-6), DOUBLE: (1e-12, 1e-13), HALF: (1e-2, 1e-2), BFLOAT16: (2e-2, 2e-2)}[dtype]
    assert_close(np.asarray(_got(got, dtype)).reshape(out_shape), np.asarray(_f(oz)).reshape(out_shape), rtol, atol, "entropy op %d dtype %d dims %s" % (op, dtype, dims))


@pytest.mark.parametrize("dtype", [FLOAT32, DOUBLE, BFLOAT16])
@pytest.mark.parametrize("dims", [[2], [0, 2], [1], None])
def test_summary_stats(ex, oracle, dtype, dims):
    from deeplearning4j_amd.executioner import SummaryStats
    rng = np.random.default_rng(70)
    x = rng.normal(100.0 if dtype != BFLOAT16 else 1.0, 2.0, (7, 9, 300))
    ox, dx = _pair(oracle, x, dtype)
    shape = () if dims is None else tuple(s for i, s in enumerate(x.shape) if i not in dims)
    for op in (SummaryStats.Variance, SummaryStats.StandardDeviation):
        for bias in (False, True):
            oz = oracle.Arr(np.zeros(shape, ox.a.dtype), ox.dt)
            oracle.summary_stats(op, ox, oz, dims, bias)
            got = ex.exec_summary_stats(op, dx, dims, bias)
            rtol = {FLOAT32: 2e-6, DOUBLE: 1e-11, BFLOAT16: 1e-2}[dtype]
            assert_close(np.asarray(_got(got, dtype)).reshape(shape), np.asarray(_f(oz)).reshape(shape), rtol, 0, "summary stats op %d bias %s dims %s" % (op, bias, dims))


def test_summary_stats_long_run_is_split_over_blocks(ex, oracle):
    from deeplearning4j_amd.executioner import SummaryStats
    rng = np.random.default_rng(71)
    x = rng.normal(50.0, 3.0, (3, 400000)).astype(np.float32)
    X = NDArray.from_numpy(x)
    want = np.var(x.astype(np.float64), axis=1, ddof=1)
    got = ex.exec_summary_stats(SummaryStats.Variance, X, [1], True).to_numpy()
    assert_close(got, want, 2e-6, 0, "variance of long rows")
    got = ex.exec_summary_stats(SummaryStats.StandardDeviation, X).to_numpy()
    assert_close(np.asarray(got).reshape(()), np.std(x.astype(np.float64)), 2e-6, 0, "std of everything")


def test_reduce_long_bool_and_transform_bool(ex, oracle):
    from deeplearning4j_amd.executioner import ReduceBool, ReduceLong, TransformBool
    from deeplearning4j_amd.ndarray import BOOL, INT64
    rng = np.random.default_rng(72)
    x = np.round(rng.normal(0, 1, (6, 50, 9))).astype(np.float32)          # many exact zeros
    X = NDArray.from_numpy(x)
    for dims in ([1], [0, 2], None):
        shape = () if dims is None else tuple(s for i, s in enumerate(x.shape) if i not in dims)
        for op in (ReduceLong.CountNonZero, ReduceLong.CountZero):
            want = oracle.reduce_long(op, x, np.zeros(shape, np.int64), dims)
            got = ex.exec_reduce_long(op, X, dims).to_numpy()
            assert np.array_equal(np.asarray(got).reshape(shape), want), (op, dims)
        for op in (ReduceBool.Any, ReduceBool.All):
            want = oracle.reduce_bool(op, x, np.zeros(shape, np.bool_), dims)
            got = ex.exec_reduce_bool(op, X, dims).to_numpy()
            assert np.array_equal(np.asarray(got).reshape(shape), want), (op, dims)
    v = np.array([0.0, -0.0, 1.0, -3.0, np.inf, -np.inf, np.nan, 1e300, 5e-324, 2.5], np.float64)
    for dt in (np.float64, np.float32):
        vv = v.astype(dt)
        V = NDArray.from_numpy(vv)
        for op in (TransformBool.IsInf, TransformBool.IsNan, TransformBool.IsFinite, TransformBool.IsInfOrNan, TransformBool.IsPositive,
                   TransformBool.Not, TransformBool.IsNegative):
            want = oracle.transform_bool(op, vv, np.zeros(vv.shape, np.bool_))
            got = ex.exec_transform_bool(op, V).to_numpy()
            assert np.array_equal(got, want), (op, dt)


@pytest.mark.parametrize("dtype", [FLOAT32, DOUBLE, BFLOAT16])
@pytest.mark.parametrize("dims", [[1], [0, 2], None])
def test_reduce3(ex, oracle, dtype, dims):
    from deeplearning4j_amd.executioner import Reduce3
    rng = np.random.default_rng(80)
    a = np.round(rng.uniform(0.25, 3, (6, 70, 5)) * 4) / 4
    b = np.round(rng.uniform(0.25, 3, (6, 70, 5)) * 4) / 4
    oa, da = _pair(oracle, a, dtype)
    ob, db = _pair(oracle, b, dtype)
    shape = () if dims is None else tuple(s for i, s in enumerate(a.shape) if i not in dims)
    for op in (Reduce3.ManhattanDistance, Reduce3.EuclideanDistance, Reduce3.CosineSimilarity, Reduce3.Dot, Reduce3.CosineDistance,
               Reduce3.JaccardDistance, Reduce3.SimpleHammingDistance):
        oz = oracle.Arr(np.zeros(shape, oa.a.dtype), oa.dt)
        oracle.reduce3(op, oa, ob, oz, dims)
        got = ex.exec_reduce3(op, da, db, dims)
        rtol, atol = {FLOAT32: (2e-6, 1e-6), DOUBLE: (1e-12, 1e-14), BFLOAT16: (1e-2, 1e-2)}[dtype]
        assert_close(np.asarray(_got(got, dtype)).reshape(shape), np.asarray(_f(oz)).reshape(shape), rtol, atol, "reduce3 op %d dims %s" % (op, dims))


def test_reduce3_reference_vectors_and_views(ex, oracle):
    from deeplearning4j_amd.executioner import Reduce3
    x = NDArray.from_numpy(np.array([[1, 2, 3], [4, 5, 6]], np.float32))
    y = NDArray.from_numpy(np.full((2, 3), 2, np.float32))
    got = ex.exec_reduce3(Reduce3.EuclideanDistance, x, y, [1]).to_numpy()        # NDArrayTests.cpp:1473-1488
    assert_close(got, [1.414214, 5.385165], 1e-6, 0, "euclidean rows")
    rng = np.random.default_rng(81)
    a = rng.normal(size=(8, 12)).astype(np.float32)
    b = rng.normal(size=(12, 8)).astype(np.float32)
    want = oracle.reduce3(Reduce3.Dot, a, b.T, np.zeros(8, np.float32), [1])
    got = ex.exec_reduce3(Reduce3.Dot, NDArray.from_numpy(a), NDArray.from_numpy(b).permute(1, 0), [1]).to_numpy()
    assert_close(got, want, 2e-6, 1e-6, "dot against a transposed view")
