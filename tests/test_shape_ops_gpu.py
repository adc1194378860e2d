"""Shape ops through the C ABI (permute, transpose, reshape, squeeze, expand_dims, split, strided_slice): index work,
so every comparison with the oracle and with the reference's own vectors is bit-exact."""
import json
import os

import numpy as np
import pytest

from deeplearning4j_amd.ndarray import BFLOAT16, DOUBLE, FLOAT32, INT32, INT64, NDArray, f32_to_bf16_bits
from deeplearning4j_amd.nativeops import NativeOpsError

pytestmark = pytest.mark.gpu

GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "strided_slice_vectors.json")))["cases"]


def _run(ex, name, inputs, **kw):
    return ex.exec_custom(name, inputs, **kw)


@pytest.mark.parametrize("case", GOLD, ids=[c["name"].split()[-1] for c in GOLD])
def test_strided_slice_reference_vectors(ex, case):
    x = NDArray.from_numpy(np.array(case["x"], dtype=np.float64))
    if "iargs" in case:
        out = _run(ex, "strided_slice", [x], i_args=case["masks"] + case["iargs"])[0]
    else:
        dt = np.float64 if case.get("float_specs") else np.int32
        specs = [NDArray.from_numpy(np.array(case["inputs"][k], dtype=dt)) for k in ("begin", "end", "strides")]
        out = _run(ex, "strided_slice", [x] + specs, i_args=case["masks"])[0]
    got = out.to_numpy()
    assert list(got.shape) == case["shape"]
    assert np.array_equal(got.reshape(-1), np.array(case["exp"], dtype=np.float64))


def test_strided_slice_random_specs_match_oracle(ex, oracle):
    rng = np.random.default_rng(1)
    x = rng.normal(size=(4, 5, 6, 3)).astype(np.float32)
    X = NDArray.from_numpy(x)
    done = 0
    for _ in range(120):
        n = int(rng.integers(1, 5))
        b = [int(rng.integers(-7, 8)) for _ in range(n)]
        e = [int(rng.integers(-7, 8)) for _ in range(n)]
        s = [int(rng.choice([-2, -1, 1, 2, 3])) for _ in range(n)]
        bm, em = int(rng.integers(0, 1 << n)), int(rng.integers(0, 1 << n))
        want = oracle.strided_slice(x, b, e, s, bm, 0, em, 0, 0)
        if want.size == 0:
            continue
        got = _run(ex, "strided_slice", [X], i_args=[bm, 0, em, 0, 0] + b + e + s)[0].to_numpy()
        assert got.shape == want.shape and np.array_equal(got, want), (b, e, s, bm, em)
        done += 1
    assert done > 40


def test_strided_slice_masks_views_and_types(ex, oracle):
    rng = np.random.default_rng(2)
    x = rng.integers(-1000, 1000, size=(3, 4, 5, 6)).astype(np.int64)
    X = NDArray.from_numpy(x)
    # x[1, ..., newaxis, ::2]  (shrink on spec 0, ellipsis on spec 1, new axis on spec 2)
    got = _run(ex, "strided_slice", [X], i_args=[0, 2, 0, 4, 1, 1, 0, 0, 0, 0, 0, 0, 6, 1, 1, 1, 2])[0].to_numpy()
    want = oracle.strided_slice(x, [1, 0, 0, 0], [0, 0, 0, 6], [1, 1, 1, 2], 0, 2, 0, 4, 1)
    assert want.shape == (4, 5, 1, 3) and np.array_equal(got, want)
    # a permuted view as the input, bf16 payload
    f = rng.normal(size=(6, 5, 4)).astype(np.float32)
    bits = f32_to_bf16_bits(f)
    V = NDArray.from_numpy(bits, BFLOAT16).permute(2, 0, 1)        # [4, 6, 5] view
    got = _run(ex, "strided_slice", [V], i_args=[0, 0, 0, 0, 0, 1, 0, 1, 3, 6, 5, 1, 2, 3])[0].to_numpy()
    want = oracle.strided_slice(bits.transpose(2, 0, 1), [1, 0, 1], [3, 6, 5], [1, 2, 3])
    assert np.array_equal(got, want)


def test_strided_slice_empty_results_and_errors(ex):
    x = NDArray.from_numpy(np.arange(10, dtype=np.float64).reshape(1, 10)[:, :1].copy().reshape(1))
    shapes = ex.calculate_output_shapes("strided_slice", [x, NDArray.from_numpy(np.array([0], np.int32)), NDArray.from_numpy(np.array([0], np.int32)),
                                                           NDArray.from_numpy(np.array([1], np.int32))], i_args=[1, 0, 0, 0, 0])
    rank = int(shapes[0][0])
    assert (int(shapes[0][2 * rank + 1 if rank else 3]) & 8) != 0          # DeclarableOpsTests4.cpp:1306-1318: an empty result
    m = NDArray.from_numpy(np.zeros((3, 4), np.float32))
    with pytest.raises(NativeOpsError, match="Number of Integer arguments"):
        ex.calculate_output_shapes("strided_slice", [m], i_args=[0, 0, 0, 0, 0, 1, 2])
    with pytest.raises(NativeOpsError, match="shape calculation failed"):
        ex.calculate_output_shapes("strided_slice", [m], i_args=[0, 0, 0, 0, 1, 5, 6, 1])      # shrink index out of range


@pytest.mark.parametrize("dtype", [FLOAT32, DOUBLE, INT32, INT64])
def test_permute_transpose_reshape(ex, oracle, dtype):
    np_dt = {FLOAT32: np.float32, DOUBLE: np.float64, INT32: np.int32, INT64: np.int64}[dtype]
    rng = np.random.default_rng(3)
    x = rng.integers(-50, 50, size=(3, 4, 5)).astype(np_dt)
    X = NDArray.from_numpy(x)
    for perm in ([2, 0, 1], [1, 0, 2], [0, 1, 2]):
        got = _run(ex, "permute", [X], i_args=perm)[0].to_numpy()
        assert np.array_equal(got, oracle.permute(x, perm))
    got = _run(ex, "permute", [X, NDArray.from_numpy(np.array([1, 2, 0], np.int32))])[0].to_numpy()
    assert np.array_equal(got, oracle.permute(x, [1, 2, 0]))
    assert np.array_equal(_run(ex, "transpose", [X])[0].to_numpy(), oracle.permute(x))
    assert np.array_equal(_run(ex, "transpose", [X], i_args=[0, 2, 1])[0].to_numpy(), oracle.permute(x, [0, 2, 1]))
    for shape in ([6, 10], [-1, 4], [2, 3, 2, 5], [60]):
        got = _run(ex, "reshape", [X], i_args=shape)[0].to_numpy()
        assert np.array_equal(got, oracle.reshape(x, shape))
    got = _run(ex, "reshape", [X], i_args=[-99, 12, 5])[0].to_numpy()
    assert np.array_equal(got, oracle.reshape(x, [12, 5]))
    got = _run(ex, "reshape", [X], i_args=[-102, 12, 5])[0]
    assert np.array_equal(got.to_numpy(), oracle.reshape(x, [12, 5], "f"))
    got = _run(ex, "reshape", [X.permute(2, 1, 0), NDArray.from_numpy(np.array([10, -1], np.int64))])[0].to_numpy()
    assert np.array_equal(got, oracle.reshape(x.transpose(2, 1, 0), [10, -1]))


@pytest.mark.parametrize("np_dt,dtype", [(np.float32, FLOAT32), (np.float64, DOUBLE), (np.float16, None), (np.uint16, BFLOAT16)])
@pytest.mark.parametrize("shape,perm,lo", [((130, 200), (1, 0), 0), ((128, 192), (1, 0), 0), ((3, 128, 256), (0, 2, 1), 0), ((2, 70, 129), (2, 0, 1), 0),
                                           ((131, 203), (1, 0), 3), ((64, 64), (1, 0), 1)])
def test_transposing_copies_whole_and_ragged_tiles(ex, np_dt, dtype, shape, perm, lo):
    """permute writes a dense copy of a view whose unit stride runs along another axis than the result's: whole 64 x 64 tiles
    move as 16-byte vectors on both sides, ragged edges element by element; `lo` cuts rows and columns off the input so that
    its rows start off 16-byte boundaries.  Bit patterns are compared (bf16 arrays are carried as their uint16 patterns)."""
    rng = np.random.default_rng(sum(shape) + lo)
    full = rng.integers(0, 60000, size=shape).astype(np.uint16)
    host = full if np_dt == np.uint16 else (full.view(np.float16) if np_dt == np.float16 else (full % 1000).astype(np_dt))
    X = NDArray.from_numpy(host, dtype) if dtype == BFLOAT16 else NDArray.from_numpy(host)
    view, want = X, host
    if lo:
        view = X.slice(len(shape) - 1, lo, shape[-1]).slice(len(shape) - 2, lo, shape[-2])
        want = host[..., lo:, lo:]
    got = _run(ex, "permute", [view], i_args=list(perm))[0].to_numpy()
    assert got.shape == tuple(want.shape[p] for p in perm)
    assert np.array_equal(got.view(np.uint8), np.ascontiguousarray(want.transpose(perm)).view(np.uint8))


def test_reshape_errors(ex):
    X = NDArray.from_numpy(np.zeros((3, 4), np.float32))
    with pytest.raises(NativeOpsError, match="Only one unknown dimension"):
        ex.calculate_output_shapes("reshape", [X], i_args=[-1, -1])
    with pytest.raises(NativeOpsError, match="lengths before and after reshape should match"):
        ex.exec_custom("reshape", [X], outputs=[NDArray.empty((5, 2), FLOAT32)], i_args=[5, 2])
    with pytest.raises(NativeOpsError, match="number of permutations"):
        ex.calculate_output_shapes("permute", [X], i_args=[0])


def test_squeeze_expand_dims_split(ex, oracle):
    rng = np.random.default_rng(4)
    x = rng.normal(size=(2, 1, 6, 1, 4)).astype(np.float32)
    X = NDArray.from_numpy(x)
    assert np.array_equal(_run(ex, "squeeze", [X])[0].to_numpy(), oracle.squeeze(x))
    assert np.array_equal(_run(ex, "squeeze", [X], i_args=[1])[0].to_numpy(), oracle.squeeze(x, [1]))
    assert np.array_equal(_run(ex, "squeeze", [X], i_args=[-2, 0])[0].to_numpy(), oracle.squeeze(x, [-2, 0]))
    y = x.reshape(2, 6, 4)
    Y = NDArray.from_numpy(y)
    for axis in (0, 2, -1):
        assert np.array_equal(_run(ex, "expand_dims", [Y], i_args=[axis])[0].to_numpy(), oracle.expand_dims(y, axis))
    for axis, parts in ((1, 3), (2, 2), (-1, 4), (0, 2)):
        outs = _run(ex, "split", [Y], i_args=[parts, axis])
        want = oracle.split(y, parts, axis)
        assert len(outs) == parts
        for o, w in zip(outs, want):
            assert np.array_equal(o.to_numpy(), w)
    outs = _run(ex, "split", [NDArray.from_numpy(np.array(1, np.int32)), Y], i_args=[2])      # axis first, as a scalar input
    assert np.array_equal(outs[1].to_numpy(), oracle.split(y, 2, 1)[1])
    with pytest.raises(NativeOpsError, match="remainder of division"):
        ex.calculate_output_shapes("split", [Y], i_args=[4, 1]); ex.exec_custom("split", [Y], i_args=[4, 1])
