"""Seeded random sweep of the legacy loops over arbitrary views: rank 1-5, axes in any memory order, gaps between
elements, offsets, zero strides on inputs, every operand with a layout of its own.  The expectation is numpy on the
logical values (one IEEE operation per element, or a selection: identical bits; sums within the re-ordering bound), so
what is under test is the shape walk of the kernels behind execPairwiseTransform / execTransformSame / execScalar /
execBroadcast / execReduceSame / execIndexReduce (reference: helpers/shape.h:588-740 INDEX2COORDS / COORDS2INDEX, which
every loop in loops/cpu/*.hpp goes through)."""
import numpy as np
import pytest

from deeplearning4j_amd.executioner import Broadcast, IndexReduce, Pairwise, ReduceSame, Scalar, TransformSame
from deeplearning4j_amd.ndarray import (BFLOAT16, DOUBLE, DT_NP, FLOAT32, HALF, INT32, INT64, DataBuffer, NDArray, bf16_bits_to_f32,
                                        f32_to_bf16_bits)
from deeplearning4j_amd import nativeops as N

pytestmark = pytest.mark.gpu

FLOATS = [FLOAT32, HALF, BFLOAT16, DOUBLE]
ALL = FLOATS + [INT32, INT64]


def logical(a, dt):
    """stored values -> the numbers they stand for (bf16 travels as bit patterns)"""
    return bf16_bits_to_f32(a) if dt == BFLOAT16 else a


def store(v, dt):
    """numbers -> stored values, rounded to nearest even where the type is narrower"""
    if dt == BFLOAT16:
        return f32_to_bf16_bits(np.asarray(v, np.float32))
    return np.asarray(v).astype(DT_NP[dt])


def random_shape(rng, max_rank=5, max_len=4000):
    while True:
        rank = int(rng.integers(1, max_rank + 1))
        shape = [int(rng.choice([1, 2, 3, 4, 5, 7, 8, 16, 17, 33, 64])) for _ in range(rank)]
        if np.prod(shape) <= max_len:
            return shape


def random_view(rng, shape, dt, values=None, writable=False):
    """A device array of `shape` laid out at random inside a larger buffer, filled with `values` (or random ones).
    Returns (NDArray, logical numpy values)."""
    rank = len(shape)
    order = list(rng.permutation(rank))                     # memory order of the axes, innermost first
    strides = [0] * rank
    run = 1
    for ax in order:
        gap = int(rng.choice([1, 1, 1, 2, 3]))
        if not writable and shape[ax] > 1 and rng.random() < 0.08:
            strides[ax] = 0                                 # a broadcast view: every index of the axis is one element
            continue
        strides[ax] = run * gap
        run = strides[ax] * shape[ax]
    offset = int(rng.integers(0, 9))
    extent = offset + sum((s - 1) * st for s, st in zip(shape, strides)) + 1
    n = extent + int(rng.integers(0, 5))
    buf = DataBuffer(n, dt)
    host = buf.host_view()
    if dt in (INT32, INT64):
        fill = rng.integers(-50, 50, n)
    else:
        fill = rng.uniform(-2, 2, n)
    host[:n] = store(fill, dt)
    arr = NDArray(buf, shape, strides, dt, offset)
    item = host.itemsize
    v = np.lib.stride_tricks.as_strided(host[offset:], shape=shape, strides=[s * item for s in strides], writeable=True)
    if values is not None:
        assert writable or 0 not in [st for s, st in zip(shape, strides) if s > 1]
        v[...] = store(values, dt).reshape(shape)
    N.load().dbTickHostWrite(buf.ptr)
    return arr, np.array(logical(np.array(v), dt)), (np.array(host[:n]), offset, strides)


def untouched_outside(arr, before):
    """the elements of the buffer that the view does not cover still hold what they held"""
    host0, offset, strides = before
    arr.to_numpy()                                          # device -> host
    host = arr.buffer.host_view()[: host0.size]
    mask = np.ones(host0.size, bool)
    idx = np.zeros(arr.shape, np.int64) + offset
    for ax, (s, st) in enumerate(zip(arr.shape, strides)):
        sh = [1] * len(arr.shape); sh[ax] = s
        idx = idx + (np.arange(s) * st).reshape(sh)
    mask[idx.ravel()] = False
    return np.array_equal(np.array(host)[mask], host0[mask])


PW = {Pairwise.Add: np.add, Pairwise.Subtract: np.subtract, Pairwise.Multiply: np.multiply}


def test_pairwise_on_random_views(ex):
    rng = np.random.default_rng(20240)
    for case in range(90):
        dt = ALL[case % len(ALL)]
        shape = random_shape(rng)
        op = list(PW)[case % 3]
        x, xv, _ = random_view(rng, shape, dt)
        y, yv, _ = random_view(rng, shape, dt)
        z, _, before = random_view(rng, shape, dt, writable=True)
        ex.exec_pairwise(op, x, y, z)
        acc = np.float64 if dt == DOUBLE else np.int64 if dt in (INT32, INT64) else np.float32
        want = store(PW[op](xv.astype(acc), yv.astype(acc)), dt)
        got = z.to_numpy()
        assert np.array_equal(got, want), "case %d: op %d dtype %d shape %s x%s y%s z%s" % (case, op, dt, shape, x.strides, y.strides, z.strides)
        assert untouched_outside(z, before), "case %d wrote outside its view" % case


def test_transform_and_scalar_on_random_views(ex):
    rng = np.random.default_rng(20241)
    for case in range(90):
        dt = ALL[case % len(ALL)]
        shape = random_shape(rng)
        x, xv, _ = random_view(rng, shape, dt)
        z, _, before = random_view(rng, shape, dt, writable=True)
        acc = np.float64 if dt == DOUBLE else np.int64 if dt in (INT32, INT64) else np.float32
        kind = case % 3
        if kind == 0:
            ex.exec_transform_same(TransformSame.Abs, x, z)
            want = store(np.abs(xv.astype(acc)), dt)
        elif kind == 1:
            ex.exec_transform_same(TransformSame.Neg, x, z)
            want = store(-xv.astype(acc), dt)
        else:
            sc = 3 if dt in (INT32, INT64) else 0.75
            ex.exec_scalar(Scalar.Add, x, NDArray.scalar(sc, dt), z)
            want = store(xv.astype(acc) + acc(sc), dt)
        assert np.array_equal(z.to_numpy(), want), "case %d: kind %d dtype %d shape %s x%s z%s" % (case, kind, dt, shape, x.strides, z.strides)
        assert untouched_outside(z, before), "case %d wrote outside its view" % case


def test_broadcast_on_random_views(ex):
    rng = np.random.default_rng(20242)
    for case in range(60):
        dt = FLOATS[case % len(FLOATS)]
        shape = random_shape(rng, max_rank=4)
        rank = len(shape)
        k = int(rng.integers(1, rank + 1))
        dims = sorted(int(d) for d in rng.choice(rank, size=k, replace=False))
        x, xv, _ = random_view(rng, shape, dt)
        y, yv, _ = random_view(rng, [shape[d] for d in dims], dt)
        z, _, before = random_view(rng, shape, dt, writable=True)
        ex.exec_broadcast(Broadcast.Add, x, y, dims, z)
        sh = [shape[d] if d in dims else 1 for d in range(rank)]
        acc = np.float64 if dt == DOUBLE else np.float32
        want = store(xv.astype(acc) + yv.astype(acc).reshape(sh), dt)
        assert np.array_equal(z.to_numpy(), want), "case %d: dtype %d shape %s dims %s" % (case, dt, shape, dims)
        assert untouched_outside(z, before), "case %d wrote outside its view" % case


def test_reductions_on_random_views(ex):
    rng = np.random.default_rng(20243)
    for case in range(90):
        dt = [FLOAT32, DOUBLE, INT32, INT64, HALF, BFLOAT16][case % 6]
        shape = random_shape(rng, max_rank=4, max_len=20000)
        rank = len(shape)
        k = int(rng.integers(0, rank + 1))
        dims = sorted(int(d) for d in rng.choice(rank, size=k, replace=False)) if k else None
        x, xv, _ = random_view(rng, shape, dt)
        zshape = [s for d, s in enumerate(shape) if dims is not None and d not in dims] if dims else []
        op = [ReduceSame.Sum, ReduceSame.Max, ReduceSame.Min][case % 3]
        if len(zshape):
            z, _, before = random_view(rng, zshape, dt, writable=True)
        else:
            z, before = NDArray.empty(zshape, dt), None
        ex.exec_reduce_same(op, x, dims, z=z)
        axes = tuple(dims) if dims else None
        got = np.asarray(logical(z.to_numpy(), dt)).reshape(np.shape(xv.sum(axis=axes)))
        if op == ReduceSame.Sum:
            if dt in (INT32, INT64):
                want = xv.astype(np.int64).sum(axis=axes).astype(DT_NP[dt])
                assert np.array_equal(got, want), "case %d: int sum shape %s dims %s" % (case, shape, dims)
            else:
                want = xv.astype(np.float64).sum(axis=axes)
                mag = np.abs(xv.astype(np.float64)).sum(axis=axes)
                eps = {FLOAT32: 2.0 ** -23, DOUBLE: 2.0 ** -52, HALF: 2.0 ** -10, BFLOAT16: 2.0 ** -7}[dt]
                n = xv.size / max(np.size(want), 1)
                assert np.all(np.abs(got - want) <= eps * (np.abs(want) + 1e-30) + (2.0 ** -23 if dt in (HALF, BFLOAT16) else eps) * n * mag), \
                    "case %d: sum dtype %d shape %s dims %s strides %s" % (case, dt, shape, dims, x.strides)
        else:
            want = (np.max if op == ReduceSame.Max else np.min)(xv, axis=axes)
            assert np.array_equal(got, want), "case %d: op %d dtype %d shape %s dims %s strides %s" % (case, op, dt, shape, dims, x.strides)
        if before is not None:
            assert untouched_outside(z, before), "case %d wrote outside its view" % case


def test_index_reduce_on_random_views(ex):
    rng = np.random.default_rng(20244)
    for case in range(60):
        dt = [FLOAT32, HALF, BFLOAT16, INT32, DOUBLE][case % 5]
        shape = random_shape(rng, max_rank=4, max_len=2000)
        rank = len(shape)
        n = int(np.prod(shape))
        # distinct values, exactly representable in every type (|v| < 2^8 in steps of 1/2 at most 2000 of them is too many for
        # bf16, so values repeat there: ties go to the lowest index, as numpy's argmax does)
        vals = rng.permutation(n).astype(np.float64) - n // 2
        if dt in (HALF, BFLOAT16):
            vals = np.round(vals / max(n / 200.0, 1.0))
        x, xv, _ = random_view(rng, shape, dt, values=vals.reshape(shape), writable=True)
        full = case % 4 == 0
        op = IndexReduce.IndexMax if case % 2 == 0 else IndexReduce.IndexMin
        if full:
            z = ex.exec_index_reduce(op, x)
            want = (np.argmax if op == IndexReduce.IndexMax else np.argmin)(xv.ravel())
            assert int(z.to_numpy()) == int(want), "case %d: full shape %s strides %s" % (case, shape, x.strides)
        else:
            d = int(rng.integers(0, rank))
            z = ex.exec_index_reduce(op, x, [d])
            want = (np.argmax if op == IndexReduce.IndexMax else np.argmin)(xv, axis=d)
            assert np.array_equal(z.to_numpy().reshape(want.shape), want), "case %d: dim %d shape %s strides %s" % (case, d, shape, x.strides)


def test_matmul_on_random_shapes_layouts_and_flags(ex):
    """matmul (ops/declarable/generic/blas/matmul.cpp:36-170: transpose flags as integer arguments, alpha and beta as
    floating ones, leading batch dimensions) over random sizes from one row to a few hundred, every combination of flags,
    operands dense or as pitched views, against numpy in fp64.  The sizes straddle every dispatch boundary of the GEMM
    (GEMV, skinny, split-K, small and large tiles, ragged edges)."""
    rng = np.random.default_rng(20245)
    sizes = [1, 2, 3, 5, 8, 17, 31, 32, 33, 64, 65, 96, 127, 128, 129, 200, 256, 257, 384]
    for case in range(72):
        dt = [FLOAT32, BFLOAT16, HALF][case % 3]
        M, N, K = (int(rng.choice(sizes)) for _ in range(3))
        ta, tb = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
        batch = [] if case % 4 else [int(rng.integers(1, 4))]
        alpha, beta = (1.0, 0.0) if case % 5 else (0.5, 2.0)
        pitched = case % 3 == 1

        def operand(rows, cols):
            shape = batch + [rows, cols]
            vals = rng.uniform(-1, 1, shape) / np.sqrt(K)
            if not pitched:
                arr = NDArray.from_numpy(store(vals, dt), dt)
                return arr, np.asarray(logical(arr.to_numpy(), dt), np.float64)
            big = NDArray.from_numpy(store(rng.uniform(-1, 1, batch + [rows + 3, cols + 8]), dt), dt)
            v = big.slice(len(batch), 1, rows + 1).slice(len(batch) + 1, 8, cols + 8)
            v.assign_numpy(store(vals, dt))
            return v, np.asarray(logical(v.to_numpy(), dt), np.float64)

        a, av = operand(K, M) if ta else operand(M, K)
        b, bv = operand(N, K) if tb else operand(K, N)
        c0 = rng.uniform(-1, 1, batch + [M, N])
        c = NDArray.from_numpy(store(c0, dt), dt)
        cv = np.asarray(logical(c.to_numpy(), dt), np.float64)
        A = np.swapaxes(av, -1, -2) if ta else av
        B = np.swapaxes(bv, -1, -2) if tb else bv
        want = alpha * (A @ B) + (beta * cv if beta else 0.0)
        ex.exec_custom("matmul", [a, b], [c], t_args=[alpha, beta], i_args=[int(ta), int(tb)])
        got = np.asarray(logical(c.to_numpy(), dt), np.float64)
        tol = {FLOAT32: 2e-6, BFLOAT16: 6e-3, HALF: 8e-4}[dt]
        bound = tol * (alpha * (np.abs(A) @ np.abs(B)) + abs(beta) * np.abs(cv) + np.abs(want)) + (6e-8 if dt == HALF else 1e-30)   # fp16: subnormal spacing
        kern = ex.L.nd4jhipLastGemmKernel().decode()
        assert np.all(np.abs(got - want) <= bound), "case %d: dtype %d M %d N %d K %d ta %d tb %d batch %s alpha %g beta %g pitched %d kernel %s: worst %g of bound" % (
            case, dt, M, N, K, ta, tb, batch, alpha, beta, pitched, kern, float(np.max(np.abs(got - want) / bound)))


def _opair(oracle, a, dt):
    if dt == BFLOAT16:
        bits = f32_to_bf16_bits(np.asarray(a, np.float32))
        return oracle.Arr(bits, oracle.BFLOAT16), NDArray.from_numpy(bits, BFLOAT16)
    h = np.asarray(a).astype(DT_NP[dt])
    return oracle.Arr(h), NDArray.from_numpy(h)


def _ozero(oracle, shape, dt):
    return oracle.Arr(np.zeros(shape, np.uint16 if dt == BFLOAT16 else DT_NP[dt]), dt)


def _ovals(oa):
    return bf16_bits_to_f32(oa.a).astype(np.float64) if oa.dt == BFLOAT16 else oa.a.astype(np.float64)


@pytest.mark.parametrize("dt,lengths", [(FLOAT32, (1028, 1280, 1536, 1540, 2048, 6144, 8192, 12288)), (DOUBLE, (516, 768, 1024, 5000)),
                                        (BFLOAT16, (2056, 2560, 3072, 3080, 4096, 12288, 16384, 16392)), (HALF, (2056, 3072, 4096, 12296))])
def test_layer_norm_rows_of_five_to_eight_wave_passes(ex, oracle, dt, lengths):
    """Rows longer than four 16-byte wave passes and up to eight stay in one wave's registers (six or eight vectors per lane,
    the last ones partly or wholly masked); longer ones take a block per row up to 8192 fp32 / 16384 16-bit elements and the
    generic kernel beyond: few rows and many, with and without bias, dense and at a pitch, against the oracle."""
    rng = np.random.default_rng(int(dt) * 7 + 1)
    rtol, atol = {FLOAT32: (2e-5, 2e-6), DOUBLE: (1e-12, 1e-12), BFLOAT16: (1e-2, 1e-2), HALF: (2e-3, 2e-3)}[dt]
    for C in lengths:
        for rows, bias, pitched in ((3, True, False), (130, False, True), (4100, True, False) if C <= 2048 else (37, True, True)):
            a = rng.normal(0.2, 1.5, (rows, C))
            ox, dx = _opair(oracle, a, dt)
            if pitched:
                wide = np.concatenate([a, rng.normal(0, 1, (rows, 16))], axis=1)
                _, dw = _opair(oracle, wide, dt)
                dx = dw.slice(1, 0, C)
            og, dg = _opair(oracle, rng.normal(1, 0.2, C), dt)
            ob, db = _opair(oracle, rng.normal(0, 0.2, C), dt)
            oz = _ozero(oracle, (rows, C), dt)
            oracle.layer_norm(ox, og, ob if bias else None, oz, [1], channels_first=False)
            z = ex.exec_custom("layer_norm", [dx, dg, db] if bias else [dx, dg], [NDArray.empty((rows, C), dt)], i_args=[1], b_args=[False])[0]
            got, want = z.to_float().astype(np.float64), _ovals(oz)
            assert np.all(np.abs(got - want) <= atol + rtol * np.abs(want)), "layer_norm rows %d x %d dtype %d bias %d pitched %d" % (rows, C, dt, bias, pitched)


@pytest.mark.parametrize("dt", [FLOAT32, DOUBLE, BFLOAT16, HALF, INT32])
def test_transposing_copies(ex, dt):
    """permute (generic/shape/permute.cpp: a strided view copied out) where the result runs along another axis than the input:
    whole and ragged 64 x 64 tiles, batches in front of and between the two axes, an input that is itself a view, and a
    result written into the middle of a larger array (nothing outside it may change).  Copies: exact."""
    rng = np.random.default_rng(int(dt) + 99)

    def make(shape):
        v = rng.integers(-100, 100, shape)
        if dt == BFLOAT16:
            return v.astype(np.float32), NDArray.from_numpy(v.astype(np.float32), BFLOAT16)
        a = v.astype(DT_NP[dt])
        return a, NDArray.from_numpy(a)

    def vals(arr):
        return arr.to_float() if dt in (BFLOAT16, HALF) else arr.to_numpy()

    for shape, perm in (((128, 192), (1, 0)), ((130, 67), (1, 0)), ((17, 1000), (1, 0)), ((3, 70, 5, 129), (0, 3, 2, 1)), ((4, 6, 100, 64), (0, 1, 3, 2)),
                        ((2, 96, 3, 80), (2, 0, 3, 1)), ((500, 257), (1, 0))):
        a, A = make(shape)
        want = np.transpose(a, perm)
        Z = NDArray.empty(want.shape, dt)
        ex.exec_custom("permute", [A], [Z], i_args=list(perm))
        assert np.array_equal(vals(Z), want.astype(vals(Z).dtype)), (shape, perm)
    # the input a column range of a wider array, the result rows 2.. and columns 3.. of a larger one
    a, A = make((150, 200))
    src = A.slice(1, 8, 8 + 130)
    want = a[:, 8:138].T
    big_np, Big = make((140, 160))
    dst = Big.slice(0, 2, 132).slice(1, 3, 153)
    ex.exec_custom("permute", [src], [dst], i_args=[1, 0])
    got = vals(Big)
    expect = big_np.astype(got.dtype).copy()
    expect[2:132, 3:153] = want.astype(got.dtype)
    assert np.array_equal(got, expect)


@pytest.mark.parametrize("dt", [FLOAT32, BFLOAT16, HALF])
def test_softmax_over_a_vocabulary(ex, oracle, dt):
    """Rows too long for a block's registers (a vocabulary's worth of logits): an odd length, so that no row after the first
    starts on a 16-byte boundary, lengths around the kernel's vector trips, a result written at a pitch of its own, and rows
    whose x and z starts differ in alignment (the element-by-element kernel)."""
    rng = np.random.default_rng(int(dt) + 50257)
    rtol, atol = {FLOAT32: (2e-5, 1e-9), BFLOAT16: (1e-2, 1e-6), HALF: (2e-3, 1e-7)}[dt]
    for rows, C in ((5, 50257), (3, 20000), (2, 131075), (4, 16385 if dt == FLOAT32 else 32770)):
        a = rng.normal(0, 2.0, (rows, C))
        a[0, C // 3] = 9.0                                   # one dominant entry
        ox, dx = _opair(oracle, a, dt)
        oz = _ozero(oracle, (rows, C), dt)
        oracle.softmax(ox, oz, 1)
        want = _ovals(oz)
        z = ex.exec_custom("softmax", [dx], [NDArray.empty((rows, C), dt)], i_args=[1])[0]
        got = z.to_float().astype(np.float64)
        assert np.all(np.abs(got - want) <= atol + rtol * np.abs(want)), "softmax rows %d x %d dtype %d" % (rows, C, dt)
        assert np.all(np.abs(got.sum(1) - 1.0) < (2e-2 if dt != FLOAT32 else 1e-4))
        # the result into columns 8.. of a wider array (another pitch, the same alignment) and into columns 3.. (another alignment)
        for first in (8, 3):
            wide = NDArray.from_numpy(np.full((rows, C + 16), 7.0, np.float32), dt) if dt == BFLOAT16 else NDArray.from_numpy(np.full((rows, C + 16), 7.0, DT_NP[dt]))
            ex.exec_custom("softmax", [dx], [wide.slice(1, first, first + C)], i_args=[1])
            w = wide.to_float().astype(np.float64)
            assert np.all(np.abs(w[:, first:first + C] - want) <= atol + rtol * np.abs(want)), "pitched result, first column %d" % first
            assert np.all(w[:, :first] == 7.0) and np.all(w[:, first + C:] == 7.0)


@pytest.mark.parametrize("dt", [FLOAT32, BFLOAT16, HALF])
def test_log_softmax_over_a_vocabulary(ex, oracle, dt):
    """log_softmax (generic/nn/activations/log_softmax.cpp: log(exp(x - max) / sum)) over rows of a vocabulary's length -- an odd
    length, so that the rows start off the 16-byte boundaries -- and of a length just past the switch to the long-row kernel,
    against the oracle's restatement."""
    rng = np.random.default_rng(int(dt) + 11)
    rtol, atol = {FLOAT32: (2e-5, 2e-5), BFLOAT16: (1e-2, 2e-2), HALF: (2e-3, 4e-3)}[dt]
    for rows, C in ((4, 50257), (3, 8200), (2, 8192)):
        a = rng.normal(0, 2.0, (rows, C))
        if dt == BFLOAT16:
            held = bf16_bits_to_f32(f32_to_bf16_bits(a.astype(np.float32)))
            dx = NDArray.from_numpy(held, BFLOAT16)
        else:
            held = a.astype(DT_NP[dt])
            dx = NDArray.from_numpy(held)
        want = oracle.log_softmax(held.astype(np.float32), 1).astype(np.float64)
        z = ex.exec_custom("log_softmax", [dx], [NDArray.empty((rows, C), dt)], i_args=[1])[0]
        got = z.to_float().astype(np.float64)
        assert np.all(np.abs(got - want) <= atol + rtol * np.abs(want)), "log_softmax rows %d x %d dtype %d" % (rows, C, dt)
        assert np.all(np.abs(np.exp(got).sum(1) - 1.0) < (5e-2 if dt != FLOAT32 else 1e-3))


ROW_LENGTHS = [1, 2, 3, 7, 8, 31, 63, 64, 65, 127, 128, 255, 256, 257, 384, 512, 640, 767, 768, 769, 1000, 1023, 1024, 1025, 1536, 2048,
               2049, 3072, 4096, 4100, 6000, 8192, 8200, 12000]


def test_row_ops_over_row_lengths_and_row_counts(ex, oracle):
    """softmax, layer_norm and gelu (helpers/cpu/softmax.cpp:260-347, generic/nn/layer_norm.cpp:35-79 over standardize.cpp:34-78,
    ops/ops.h GELU) for every row length around the switch points of the row kernels (rows held in one wave's registers, in
    one block, walked in pieces), few and many rows (the layer_norm for many rows is a kernel of its own), dense and pitched
    rows, against the CPU oracle."""
    rng = np.random.default_rng(20246)
    case = 0
    for C in ROW_LENGTHS:
        for rows in ([3, 37] if C > 2048 else [1, 5, 37, 4097 if C <= 1024 else 130]):
            dt = [FLOAT32, BFLOAT16, HALF][case % 3]
            case += 1
            rtol, atol = {FLOAT32: (2e-5, 2e-6), BFLOAT16: (1e-2, 1e-2), HALF: (2e-3, 2e-3)}[dt]
            a = rng.normal(0, 1.5, (rows, C))
            ox, dx = _opair(oracle, a, dt)
            if case % 4 == 0 and C >= 8:               # pitched rows: a column slice of a wider array
                wide = np.concatenate([rng.normal(0, 1, (rows, 8)), a, rng.normal(0, 1, (rows, 8))], axis=1)
                _, dw = _opair(oracle, wide, dt)
                dx = dw.slice(1, 8, 8 + C)
            tag = "rows %d x %d dtype %d pitched %d" % (rows, C, dt, case % 4 == 0 and C >= 8)
            # softmax along the rows
            oz = _ozero(oracle, (rows, C), dt)
            oracle.softmax(ox, oz, 1)
            z = ex.exec_custom("softmax", [dx], [NDArray.empty((rows, C), dt)], i_args=[1])[0]
            got, want = z.to_float().astype(np.float64), _ovals(oz)
            assert np.all(np.abs(got - want) <= atol * 1e-2 + rtol * np.abs(want)), "softmax " + tag
            # layer_norm with gain and bias
            g, b = rng.normal(1, 0.2, C), rng.normal(0, 0.2, C)
            og, dg = _opair(oracle, g, dt)
            ob, db = _opair(oracle, b, dt)
            oz = _ozero(oracle, (rows, C), dt)
            oracle.layer_norm(ox, og, ob, oz, [1], channels_first=False)
            if C > 1:                                   # one element: the reference divides 0 by a zero deviation
                z = ex.exec_custom("layer_norm", [dx, dg, db], [NDArray.empty((rows, C), dt)], i_args=[1], b_args=[False])[0]
                got, want = z.to_float().astype(np.float64), _ovals(oz)
                assert np.all(np.abs(got - want) <= atol + rtol * np.abs(want)), "layer_norm " + tag
            # gelu
            from deeplearning4j_amd.executioner import TransformStrict
            oz = _ozero(oracle, (rows, C), dt)
            oracle.transform_strict(TransformStrict.GELU, ox, oz)
            z = ex.exec_transform_strict(TransformStrict.GELU, dx, NDArray.empty((rows, C), dt))
            got, want = z.to_float().astype(np.float64), _ovals(oz)
            assert np.all(np.abs(got - want) <= atol * 1e-1 + rtol * np.abs(want)), "gelu " + tag


def test_attention_on_random_shapes_masks_and_layouts(ex, oracle):
    """dot_product_attention_v2, output only (the fused tile kernel, the streaming kernel for a handful of query rows, or the
    composition for head sizes the fused kernels do not take): random batch, lengths from one key to a few tiles with ragged
    ends, head sizes 32 / 64 / 128, causal or not, with and without a value mask, operands dense or as token-major head
    views [T, heads, D] -> [heads, T, D], against the oracle's literal composition (AttentionHelper.cpp:189-241, 340-352).
    bf16 at head size 128 is held to 2.5 times the gate: the composition itself is that far from the exact result."""
    import math
    rng = np.random.default_rng(20247)
    for case in range(48):
        dt = [BFLOAT16, HALF][case % 2]
        D = [64, 64, 128, 32][case % 4]
        B = int(rng.integers(1, 4))
        Tq = int(rng.choice([1, 2, 5, 8, 9, 31, 64, 65, 127, 128, 129, 200, 257, 300]))
        Tv = int(rng.choice([1, 3, 63, 64, 65, 100, 128, 191, 192, 193, 320, 400]))
        causal = bool(rng.integers(0, 2))
        masked = case % 3 == 0
        views = case % 5 == 1
        scale = [1 / math.sqrt(D), 0.11, 1.0][case % 3]

        def operand(T):
            vals = rng.normal(0, 1, (B, T, D))
            if not views:
                return _opair(oracle, vals, dt) + (None,)
            tok = np.ascontiguousarray(vals.transpose(1, 0, 2))          # [T, heads, D] in memory
            o, d = _opair(oracle, tok, dt)
            return oracle.Arr(np.ascontiguousarray(o.a.transpose(1, 0, 2)), o.dt), d.permute(1, 0, 2), d
        oq, dq, _k1 = operand(Tq)
        ok, dk, _k2 = operand(Tv)
        ov, dv, _k3 = operand(Tv)
        oo, ow, ol = _ozero(oracle, (B, Tq, D), dt), _ozero(oracle, (B, Tq, Tv), dt), _ozero(oracle, (B, Tq, Tv), dt)
        ins = [dq, dv, dk]
        kw = {}
        if masked:
            vm = (rng.random((B, Tv)) > 0.4).astype(np.float32)
            vm[:, 0] = 1
            ovm, dvm = _opair(oracle, vm, dt)
            kw["v_mask"] = ovm
            ins = [dq, dv, dk, NDArray.empty((0,), dt), dvm]
        oracle.attention_v2(oq, ov, ok, oo, ow, ol, scale=scale, causal=causal, **kw)
        out = ex.exec_custom("dot_product_attention_v2", ins, [NDArray.empty((B, Tq, D), dt)], t_args=[scale, 0.0], b_args=[causal, False])[0]
        got, want = out.to_float().astype(np.float64), _ovals(oo)
        tol = 1e-2 if dt == BFLOAT16 else 2e-3
        tag = "case %d: dtype %d B %d Tq %d Tv %d D %d causal %d masked %d views %d scale %g" % (case, dt, B, Tq, Tv, D, causal, masked, views, scale)
        # the composition rounds every intermediate to the storage type and is itself some way from the exact result (at bf16
        # up to 0.02 on single elements): the kernel must stay within 2.5 times the gate of the composition and must not be
        # further from the exact result than the composition is
        assert np.all(np.abs(got - want) <= 2.5 * tol * (1 + np.abs(want))), tag + ": worst %g against the composition" % float(np.abs(got - want).max())
        q64, k64, v64 = _ovals(oq), _ovals(ok), _ovals(ov)
        sc64 = np.clip(np.einsum("bqd,bkd->bqk", q64, k64) * scale, -1e4, 1e4)
        hide = np.zeros((B, Tq, Tv), bool)
        if causal:
            hide |= ~np.tril(np.ones((Tq, Tv), bool))[None]
        if masked:
            hide |= (vm == 0)[:, None, :]
        sc64 = np.where(hide, -np.inf, sc64)
        p64 = np.exp(sc64 - sc64.max(-1, keepdims=True))
        truth = np.einsum("bqk,bkd->bqd", p64 / p64.sum(-1, keepdims=True), v64)
        assert np.abs(got - truth).max() <= 1.25 * np.abs(want - truth).max() + tol / 4, tag + ": %g from the exact result, the composition %g" % (
            float(np.abs(got - truth).max()), float(np.abs(want - truth).max()))


@pytest.mark.gpu
def test_dense_casts_between_fp32_and_the_16_bit_types(ex):
    """cast (generic/datatypes/cast.cpp -> NDArray::assign between two types, helpers/Loops.h: a static_cast per element, through
    float for the 16-bit types): lengths that are whole vectors of eight, lengths with a rest, and fewer than eight; fp32 -> f16
    and f16 <-> f16-representable values against numpy's round-to-nearest-even, fp32 -> bf16 against the bit-level rounding,
    the widening casts exact."""
    rng = np.random.default_rng(515)
    for n in (1, 5, 8, 64, 1000, 4096 * 3 + 7, 1 << 18):
        v = rng.normal(0, 30, n).astype(np.float32)
        v[:: max(1, n // 7)] = 0.0
        A = NDArray.from_numpy(v)
        h = ex.exec_custom("cast", [A], d_args=[HALF])[0]
        assert np.array_equal(h.to_numpy(), v.astype(np.float16)), n
        b = ex.exec_custom("cast", [A], d_args=[BFLOAT16])[0]
        assert np.array_equal(b.to_numpy(), f32_to_bf16_bits(v)), n
        assert np.array_equal(ex.exec_custom("cast", [h], d_args=[FLOAT32])[0].to_numpy(), v.astype(np.float16).astype(np.float32)), n
        assert np.array_equal(ex.exec_custom("cast", [b], d_args=[FLOAT32])[0].to_numpy(), bf16_bits_to_f32(f32_to_bf16_bits(v))), n
        # 16-bit to 16-bit goes through float: the bf16 values are exact in fp32, then rounded to f16
        hb = ex.exec_custom("cast", [b], d_args=[HALF])[0]
        assert np.array_equal(hb.to_numpy(), bf16_bits_to_f32(f32_to_bf16_bits(v)).astype(np.float16)), n
        bh = ex.exec_custom("cast", [h], d_args=[BFLOAT16])[0]
        assert np.array_equal(bh.to_numpy(), f32_to_bf16_bits(v.astype(np.float16).astype(np.float32))), n


@pytest.mark.gpu
@pytest.mark.parametrize("dt", [FLOAT32, HALF, BFLOAT16, DOUBLE])
def test_scalar_ops_on_dense_arrays_and_on_column_ranges(ex, dt):
    """execScalar (legacy_ops.h SCALAR_OPS, loops/cpu/scalar.hpp): the same values laid out three ways -- a dense array (16 bytes
    per thread, the rest one by one), a column range of a wider array whose rows start on 16-byte boundaries, and a range that
    starts one element off (element by element) -- must give the same bits; fp32 and double also equal numpy's.  Nothing
    outside a range written to may change."""
    rng = np.random.default_rng(616 + int(dt))
    for rows, cols in ((1, 5), (1, 1003), (37, 64), (200, 136), (3, 8)):
        vals = rng.normal(0, 3, (rows, cols)).astype(np.float32)
        wide = rng.normal(0, 3, (rows, cols + 24)).astype(np.float32)
        wide[:, 8:8 + cols] = vals
        wide1 = rng.normal(0, 3, (rows, cols + 24)).astype(np.float32)
        wide1[:, 9:9 + cols] = vals
        for op, f in ((Scalar.Multiply, lambda a: a * a.dtype.type(1.5)), (Scalar.Add, lambda a: a + a.dtype.type(0.25)),
                      (Scalar.ReverseSubtract, lambda a: a.dtype.type(2.0) - a)):
            D = NDArray.from_numpy(vals, dt)
            W = NDArray.from_numpy(wide, dt)
            W1 = NDArray.from_numpy(wide1, dt)
            zd = ex.exec_scalar(op, D, 1.5 if op == Scalar.Multiply else 0.25 if op == Scalar.Add else 2.0)
            sc = 1.5 if op == Scalar.Multiply else 0.25 if op == Scalar.Add else 2.0
            before, before1 = W.to_numpy().copy(), W1.to_numpy().copy()
            ex.exec_scalar(op, W.slice(1, 8, 8 + cols), sc, z=W.slice(1, 8, 8 + cols))
            ex.exec_scalar(op, W1.slice(1, 9, 9 + cols), sc, z=W1.slice(1, 9, 9 + cols))
            got = zd.to_numpy()
            after, after1 = W.to_numpy(), W1.to_numpy()
            assert np.array_equal(after[:, 8:8 + cols], got), (rows, cols, op)
            assert np.array_equal(after1[:, 9:9 + cols], got), (rows, cols, op)
            before[:, 8:8 + cols] = got
            before1[:, 9:9 + cols] = got
            assert np.array_equal(after, before) and np.array_equal(after1, before1), (rows, cols, op)
            if dt in (FLOAT32, DOUBLE):
                assert np.array_equal(got, f(D.to_numpy())), (rows, cols, op)


@pytest.mark.gpu
@pytest.mark.parametrize("dt", [FLOAT32, BFLOAT16, DOUBLE])
def test_gather_rows_of_whole_and_ragged_16_byte_units(ex, dt):
    """gather along axis 0 (generic/transforms/gather.cpp, helpers/cpu/gather.cpp: row idx[i] of the table becomes row i): rows
    that are whole 16-byte units move as such, others element by element; negative ids count from the end.  Copies: exact."""
    rng = np.random.default_rng(717 + int(dt))
    for rows, cols, n in ((50, 8, 33), (50, 12, 33), (1000, 768, 257), (7, 1, 20), (64, 100, 5)):
        t = rng.integers(-100, 100, (rows, cols)).astype(np.float32)
        T = NDArray.from_numpy(t, dt)
        for idt in (np.int32, np.int64):
            idx = rng.integers(-rows, rows, n).astype(idt)
            g = ex.exec_custom("gather", [T, NDArray.from_numpy(idx)], i_args=[0])[0]
            assert np.array_equal(g.to_numpy(), T.to_numpy()[idx]), (rows, cols, n, idt)
