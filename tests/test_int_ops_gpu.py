"""Integer and bool arrays on the legacy loops and the custom ops built on them, bit for bit against numpy's integer
arithmetic (the reference instantiates these loops for every common type:
libnd4j/include/legacy/cpu/NativeOpExecutioner_pairwise_floats.cpp:23-68, loops/cpu/reduce/reduce_same.hpp:156-193,
loops/cpu/indexreduce.hpp:98-140).  Wrap-around on overflow is part of the contract (C++ integer arithmetic in the
array's type)."""
import numpy as np
import pytest

from deeplearning4j_amd.executioner import Broadcast, IndexReduce, Pairwise, ReduceSame, Scalar, TransformBool, TransformSame
from deeplearning4j_amd.nativeops import NativeOpsError
from deeplearning4j_amd.ndarray import BOOL, FLOAT32, INT8, INT16, INT32, INT64, UINT8, UINT16, UINT32, UINT64, NDArray

pytestmark = pytest.mark.gpu

NP = {INT32: np.int32, INT64: np.int64}


def _draw(rng, shape, dt, wide=False):
    info = np.iinfo(NP[dt])
    if wide:   # values whose sums and products wrap around
        return rng.integers(info.min, info.max, shape, dtype=NP[dt], endpoint=True)
    return rng.integers(-1000, 1000, shape, dtype=NP[dt])


def _trunc_div(a, b):
    q = np.abs(a.astype(np.int64)) // np.abs(b.astype(np.int64))
    return (q * np.sign(a.astype(np.int64)) * np.sign(b.astype(np.int64))).astype(a.dtype)


PAIRWISE = [
    (Pairwise.Add, lambda a, b: a + b), (Pairwise.Subtract, lambda a, b: a - b), (Pairwise.Multiply, lambda a, b: a * b),
    (Pairwise.CopyPws, lambda a, b: b), (Pairwise.ReverseSubtract, lambda a, b: b - a), (Pairwise.MaxPairwise, np.maximum),
    (Pairwise.MinPairwise, np.minimum), (Pairwise.SquaredSubtract, lambda a, b: (a - b) * (a - b)),
    (Pairwise.Divide, _trunc_div), (Pairwise.FloorDiv, lambda a, b: a // b), (Pairwise.FloorMod, np.mod), (Pairwise.Mod, np.fmod),
    (Pairwise.LogicalAnd, lambda a, b: a & b), (Pairwise.LogicalOr, lambda a, b: a | b), (Pairwise.LogicalXor, lambda a, b: a ^ b),
]


@pytest.mark.parametrize("dt", [INT32, INT64])
@pytest.mark.parametrize("op,fn", PAIRWISE, ids=[str(p[0]) for p in PAIRWISE])
def test_pairwise_int(ex, dt, op, fn):
    rng = np.random.default_rng(op * 7 + dt)
    wide = op in (Pairwise.Add, Pairwise.Subtract, Pairwise.Multiply, Pairwise.SquaredSubtract, Pairwise.ReverseSubtract)
    a = _draw(rng, (257, 129), dt, wide)
    b = _draw(rng, (257, 129), dt, wide)
    if op in (Pairwise.Divide, Pairwise.FloorDiv, Pairwise.FloorMod, Pairwise.Mod):
        b[b == 0] = 7
    with np.errstate(over="ignore"):
        want = fn(a, b).astype(NP[dt])
    A, B = NDArray.from_numpy(a), NDArray.from_numpy(b)
    assert np.array_equal(ex.exec_pairwise(op, A, B).to_numpy(), want)
    # strided operands: the transposed problem through permuted views
    At, Bt = NDArray.from_numpy(np.ascontiguousarray(a.T)).permute(1, 0), NDArray.from_numpy(np.ascontiguousarray(b.T)).permute(1, 0)
    assert np.array_equal(ex.exec_pairwise(op, At, Bt, NDArray.empty(a.shape, dt)).to_numpy(), want)


def test_pairwise_bool_and_mixed_widths(ex):
    rng = np.random.default_rng(3)
    a, b = rng.integers(0, 2, 1000).astype(bool), rng.integers(0, 2, 1000).astype(bool)
    A, B = NDArray.from_numpy(a), NDArray.from_numpy(b)
    assert np.array_equal(ex.exec_pairwise(Pairwise.LogicalAnd, A, B).to_numpy(), a & b)
    assert np.array_equal(ex.exec_pairwise(Pairwise.LogicalOr, A, B).to_numpy(), a | b)
    assert np.array_equal(ex.exec_pairwise(Pairwise.LogicalXor, A, B).to_numpy(), a ^ b)
    # INT64 + INT32 -> INT64 (x or y carries z's type)
    x, y = _draw(rng, (300,), INT64), _draw(rng, (300,), INT32)
    z = ex.exec_pairwise(Pairwise.Add, NDArray.from_numpy(x), NDArray.from_numpy(y), NDArray.empty((300,), INT64)).to_numpy()
    assert np.array_equal(z, x + y)
    # a float result from integer operands
    zf = ex.exec_pairwise(Pairwise.Multiply, NDArray.from_numpy(x.astype(np.float32)), NDArray.from_numpy(y), NDArray.empty((300,), FLOAT32)).to_numpy()
    assert np.array_equal(zf, x.astype(np.float32) * y.astype(np.float32))


@pytest.mark.parametrize("dt", [INT32, INT64])
def test_scalar_broadcast_and_transform_same_int(ex, dt):
    rng = np.random.default_rng(dt)
    a = _draw(rng, (64, 48), dt)
    A = NDArray.from_numpy(a)
    for op, fn in ((Scalar.Add, lambda v: v + 13), (Scalar.Subtract, lambda v: v - 13), (Scalar.Multiply, lambda v: v * 13),
                   (Scalar.ReverseSubtract, lambda v: 13 - v), (Scalar.MaxPairwise, lambda v: np.maximum(v, 13)), (Scalar.FloorMod, lambda v: np.mod(v, 13)),
                   (Scalar.CopyPws, lambda v: np.full_like(v, 13))):
        assert np.array_equal(ex.exec_scalar(op, A, 13).to_numpy(), fn(a).astype(NP[dt])), op
    if dt == INT64:   # a scalar beyond 2^53 stays exact
        big = (1 << 60) + 1
        assert np.array_equal(ex.exec_scalar(Scalar.Add, A, NDArray.scalar(big, INT64)).to_numpy(), a + big)
    row = _draw(rng, (48,), dt)
    col = _draw(rng, (64,), dt)
    assert np.array_equal(ex.exec_broadcast(Broadcast.Add, A, NDArray.from_numpy(row), [1]).to_numpy(), a + row)
    assert np.array_equal(ex.exec_broadcast(Broadcast.Multiply, A, NDArray.from_numpy(col), [0]).to_numpy(), a * col[:, None])
    for op, fn in ((TransformSame.Abs, np.abs), (TransformSame.Neg, np.negative), (TransformSame.Square, np.square), (TransformSame.Cube, lambda v: v * v * v),
                   (TransformSame.OneMinus, lambda v: 1 - v), (TransformSame.Identity, lambda v: v), (TransformSame.Ones, np.ones_like),
                   (TransformSame.Floor, lambda v: v)):
        assert np.array_equal(ex.exec_transform_same(op, A).to_numpy(), fn(a).astype(NP[dt])), op
    assert np.array_equal(ex.exec_transform_bool(TransformBool.IsPositive, A).to_numpy(), a > 0)
    assert np.array_equal(ex.exec_transform_bool(TransformBool.Not, A).to_numpy(), a == 0)
    # assign between integer widths and into a strided view
    Z = NDArray.empty((48, 64), INT64 if dt == INT32 else INT32)
    ex.exec_assign(A, Z.permute(1, 0))
    assert np.array_equal(Z.to_numpy(), a.T.astype(np.int64 if dt == INT32 else np.int32))


@pytest.mark.parametrize("dt", [INT32, INT64])
def test_reduce_same_int(ex, dt):
    rng = np.random.default_rng(40 + dt)
    a = _draw(rng, (37, 50, 11), dt, wide=True)
    A = NDArray.from_numpy(a)
    with np.errstate(over="ignore"):
        for dims in ([2], [0], [0, 2], [1]):
            ax = tuple(dims)
            assert np.array_equal(ex.exec_reduce_same(ReduceSame.Sum, A, dims).to_numpy(), a.sum(ax, dtype=NP[dt]))
            assert np.array_equal(ex.exec_reduce_same(ReduceSame.Max, A, dims).to_numpy(), a.max(ax))
            assert np.array_equal(ex.exec_reduce_same(ReduceSame.Min, A, dims).to_numpy(), a.min(ax))
            assert np.array_equal(ex.exec_reduce_same(ReduceSame.Prod, A, dims).to_numpy(), a.prod(ax, dtype=NP[dt]))
        # full reductions, long enough to be split over many blocks
        big = _draw(rng, (3_000_017,), dt, wide=True)
        Bg = NDArray.from_numpy(big)
        assert ex.exec_reduce_same(ReduceSame.Sum, Bg, None).to_numpy() == big.sum(dtype=NP[dt])
        assert ex.exec_reduce_same(ReduceSame.Max, Bg, None).to_numpy() == big.max()
        assert ex.exec_reduce_same(ReduceSame.Min, Bg, None).to_numpy() == big.min()
        small = _draw(rng, (3_000_017,), dt)
        assert ex.exec_reduce_same(ReduceSame.ASum, NDArray.from_numpy(small), None).to_numpy() == np.abs(small).sum(dtype=NP[dt])


@pytest.mark.parametrize("dt", [INT32, INT64])
def test_index_reduce_int_first_extreme_wins(ex, dt):
    rng = np.random.default_rng(50 + dt)
    a = rng.integers(-5, 6, (64, 777)).astype(NP[dt])          # few distinct values: every row has ties
    A = NDArray.from_numpy(a)
    assert np.array_equal(ex.exec_index_reduce(IndexReduce.IndexMax, A, [1]).to_numpy(), a.argmax(1))
    assert np.array_equal(ex.exec_index_reduce(IndexReduce.IndexMin, A, [1]).to_numpy(), a.argmin(1))
    assert np.array_equal(ex.exec_index_reduce(IndexReduce.IndexAbsoluteMax, A, [1]).to_numpy(), np.abs(a).argmax(1))
    assert np.array_equal(ex.exec_index_reduce(IndexReduce.IndexAbsoluteMin, A, [0]).to_numpy(), np.abs(a).argmin(0))
    big = rng.integers(-1000, 1000, 2_500_003).astype(NP[dt])   # split over blocks; the extreme repeats across segments
    Bg = NDArray.from_numpy(big)
    assert ex.exec_index_reduce(IndexReduce.IndexMax, Bg, None).to_numpy() == big.argmax()
    assert ex.exec_index_reduce(IndexReduce.IndexMin, Bg, None).to_numpy() == big.argmin()
    z32 = ex.exec_index_reduce(IndexReduce.IndexMax, A, [1], z=NDArray.empty((64,), INT32)).to_numpy()
    assert z32.dtype == np.int32 and np.array_equal(z32, a.argmax(1))


def _u64(rng, shape):
    """Half of the values at 2^63 and above, where a signed reading of the same bits is negative."""
    a = rng.integers(0, 1 << 63, shape, dtype=np.uint64)
    a[rng.random(shape) < 0.5] |= np.uint64(1 << 63)
    a.flat[:4] = [np.uint64(1 << 63), np.uint64((1 << 64) - 1), np.uint64((1 << 63) + 1), np.uint64(0)]
    return a


def test_uint64_wraps_where_the_sign_does_not_matter(ex):
    """UINT64 operands travel through 64-bit two's-complement arithmetic: sums, differences, products and bit ops are the
    unsigned results modulo 2^64, also for values of 2^63 and above."""
    rng = np.random.default_rng(64)
    a, b = _u64(rng, (129, 257)), _u64(rng, (129, 257))
    A, B = NDArray.from_numpy(a), NDArray.from_numpy(b)
    assert A.dtype == UINT64
    with np.errstate(over="ignore"):
        for op, fn in ((Pairwise.Add, lambda u, v: u + v), (Pairwise.Subtract, lambda u, v: u - v), (Pairwise.Multiply, lambda u, v: u * v),
                       (Pairwise.ReverseSubtract, lambda u, v: v - u), (Pairwise.SquaredSubtract, lambda u, v: (u - v) * (u - v)),
                       (Pairwise.CopyPws, lambda u, v: v), (Pairwise.LogicalAnd, lambda u, v: u & v), (Pairwise.LogicalOr, lambda u, v: u | v),
                       (Pairwise.LogicalXor, lambda u, v: u ^ v)):
            z = ex.exec_pairwise(op, A, B).to_numpy()
            assert z.dtype == np.uint64 and np.array_equal(z, fn(a, b)), op
        # strided operands and a narrower unsigned y, which is read without sign extension
        At = NDArray.from_numpy(np.ascontiguousarray(a.T)).permute(1, 0)
        y32 = rng.integers(1 << 31, 1 << 32, a.shape, dtype=np.uint32)
        z = ex.exec_pairwise(Pairwise.Add, At, NDArray.from_numpy(y32), NDArray.empty(a.shape, UINT64)).to_numpy()
        assert np.array_equal(z, a + y32.astype(np.uint64))
        for op, fn in ((TransformSame.Neg, lambda u: np.uint64(0) - u), (TransformSame.Square, lambda u: u * u), (TransformSame.Cube, lambda u: u * u * u),
                       (TransformSame.OneMinus, lambda u: np.uint64(1) - u), (TransformSame.Identity, lambda u: u), (TransformSame.Ones, np.ones_like)):
            assert np.array_equal(ex.exec_transform_same(op, A).to_numpy(), fn(a)), op
        assert np.array_equal(ex.exec_transform_bool(TransformBool.Not, A).to_numpy(), a == 0)
        for dims in ([1], [0], None):
            ax = None if dims is None else tuple(dims)
            assert np.array_equal(ex.exec_reduce_same(ReduceSame.Sum, A, dims).to_numpy(), a.sum(ax, dtype=np.uint64))
            assert np.array_equal(ex.exec_reduce_same(ReduceSame.Prod, A, dims).to_numpy(), a.prod(ax, dtype=np.uint64))
        big = _u64(rng, (3_000_017,))        # split over many blocks
        assert ex.exec_reduce_same(ReduceSame.Sum, NDArray.from_numpy(big), None).to_numpy() == big.sum(dtype=np.uint64)
    Z = NDArray.empty((257, 129), UINT64)
    ex.exec_assign(A, Z.permute(1, 0))
    assert np.array_equal(Z.to_numpy(), a.T)


def test_uint64_is_refused_where_a_signed_reading_would_be_wrong(ex):
    """Ordering, division, remainders, absolute values and scalar operands would treat 2^63 and above as negative numbers: the
    library raises instead, and leaves z as it was."""
    rng = np.random.default_rng(65)
    a, b = _u64(rng, (40, 33)), _u64(rng, (40, 33))
    b[b == 0] = 3
    A, B = NDArray.from_numpy(a), NDArray.from_numpy(b)
    for op in (Pairwise.Divide, Pairwise.FloorDiv, Pairwise.FloorMod, Pairwise.Mod, Pairwise.MaxPairwise, Pairwise.MinPairwise, Pairwise.TruncateDiv,
               Pairwise.AMaxPairwise, Pairwise.ReverseDivide):
        Z = NDArray.from_numpy(np.full(a.shape, 7, np.uint64))
        with pytest.raises(NativeOpsError):
            ex.exec_pairwise(op, A, B, Z)
        assert np.array_equal(Z.to_numpy(), np.full(a.shape, 7, np.uint64)), op
    for op in (Scalar.Add, Scalar.Multiply, Scalar.MaxPairwise, Scalar.Divide):
        with pytest.raises(NativeOpsError):
            ex.exec_scalar(op, A, NDArray.from_numpy(np.array(1 << 63, np.uint64)))
    for op in (TransformSame.Abs, TransformSame.Reciprocal):
        with pytest.raises(NativeOpsError):
            ex.exec_transform_same(op, A)
    for op in (TransformBool.IsPositive, TransformBool.IsNegative):
        with pytest.raises(NativeOpsError):
            ex.exec_transform_bool(op, A)
    for op in (ReduceSame.Max, ReduceSame.Min, ReduceSame.ASum, ReduceSame.AMax, ReduceSame.AMin):
        with pytest.raises(NativeOpsError):
            ex.exec_reduce_same(op, A, [1])
        with pytest.raises(NativeOpsError):
            ex.exec_reduce_same(op, A, None)
    for op in (IndexReduce.IndexMax, IndexReduce.IndexMin, IndexReduce.IndexAbsoluteMax):
        with pytest.raises(NativeOpsError):
            ex.exec_index_reduce(op, A, [1])
    # the library still works afterwards
    with np.errstate(over="ignore"):
        assert np.array_equal(ex.exec_pairwise(Pairwise.Add, A, B).to_numpy(), a + b)


@pytest.mark.parametrize("dt,npdt", [(INT8, np.int8), (UINT8, np.uint8), (INT16, np.int16), (UINT16, np.uint16), (UINT32, np.uint32)])
def test_narrow_and_unsigned_integer_types(ex, dt, npdt):
    """The narrow types are widened to 64 bits on the way in (with or without sign, as the type says) and cut back on the way
    out, so that every op, ordering and division included, sees the values the type holds."""
    rng = np.random.default_rng(70 + dt)
    info = np.iinfo(npdt)
    a = rng.integers(info.min, info.max, (130, 67), dtype=npdt, endpoint=True)
    b = rng.integers(info.min, info.max, (130, 67), dtype=npdt, endpoint=True)
    a.flat[:2] = [info.max, info.min]
    b.flat[:2] = [info.max, info.max]
    bd = b.copy()
    bd[bd == 0] = 5
    A, B, Bd = NDArray.from_numpy(a), NDArray.from_numpy(b), NDArray.from_numpy(bd)
    assert A.dtype == dt
    wide = lambda v: v.astype(np.int64)
    with np.errstate(over="ignore"):
        for op, want in ((Pairwise.Add, (wide(a) + wide(b)).astype(npdt)), (Pairwise.Multiply, (wide(a) * wide(b)).astype(npdt)),
                         (Pairwise.Subtract, (wide(a) - wide(b)).astype(npdt)), (Pairwise.MaxPairwise, np.maximum(a, b)),
                         (Pairwise.MinPairwise, np.minimum(a, b))):
            z = ex.exec_pairwise(op, A, B).to_numpy()
            assert z.dtype == npdt and np.array_equal(z, want), op
        assert np.array_equal(ex.exec_pairwise(Pairwise.Divide, A, Bd).to_numpy(), _trunc_div(wide(a), wide(bd)).astype(npdt))
        assert np.array_equal(ex.exec_pairwise(Pairwise.FloorMod, A, Bd).to_numpy(), np.mod(wide(a), wide(bd)).astype(npdt))
        assert np.array_equal(ex.exec_reduce_same(ReduceSame.Sum, A, [1]).to_numpy(), wide(a).sum(1).astype(npdt))
        assert np.array_equal(ex.exec_reduce_same(ReduceSame.Max, A, [0]).to_numpy(), a.max(0))
        assert np.array_equal(ex.exec_reduce_same(ReduceSame.Min, A, None).to_numpy(), a.min())
    assert np.array_equal(ex.exec_index_reduce(IndexReduce.IndexMax, A, [1]).to_numpy(), a.argmax(1))
    assert np.array_equal(ex.exec_index_reduce(IndexReduce.IndexMin, A, [0]).to_numpy(), a.argmin(0))
    assert np.array_equal(ex.exec_scalar(Scalar.Add, A, 3).to_numpy(), (wide(a) + 3).astype(npdt))


def test_custom_ops_on_integer_arrays(ex):
    """What a decoder graph does with integers: position ids = arange + offset, arg-max over integer scores."""
    pos = np.arange(1024, dtype=np.int64).reshape(1, 1024)
    off = np.array([[17], [400]], dtype=np.int64)
    z = ex.exec_custom("add", [NDArray.from_numpy(pos), NDArray.from_numpy(off)])[0]
    assert z.dtype == INT64 and np.array_equal(z.to_numpy(), pos + off)
    scores = np.random.default_rng(1).integers(0, 50, (8, 300)).astype(np.int32)
    am = ex.exec_custom("argmax", [NDArray.from_numpy(scores)], i_args=[1])[0]
    assert np.array_equal(am.to_numpy(), scores.argmax(1))
    m = ex.exec_custom("reduce_max", [NDArray.from_numpy(scores)], i_args=[1])[0]
    assert m.dtype == INT32 and np.array_equal(m.to_numpy(), scores.max(1))
    with pytest.raises(NativeOpsError, match="not implemented for integer"):
        ex.exec_pairwise(Pairwise.Pow, NDArray.from_numpy(scores), NDArray.from_numpy(scores))
