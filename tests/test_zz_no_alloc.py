"""The entry point that allocates nothing (nd4jhipReduceSameScalarNoAlloc) against execReduceSame: same kernels, so the
same bits -- on two calls in a row, the second on a smaller input (the fixed partials array keeps the first call's
contents), for every opNum and float type, and on a caller-owned stream."""
import numpy as np
import pytest

from deeplearning4j_amd import nativeops as N
from deeplearning4j_amd.executioner import ReduceSame
from deeplearning4j_amd.ndarray import BFLOAT16, DOUBLE, FLOAT32, HALF, NDArray, f32_to_bf16_bits

pytestmark = pytest.mark.gpu


def _device(a, dt):
    if dt == BFLOAT16:
        return NDArray.from_numpy(f32_to_bf16_bits(a.astype(np.float32)), BFLOAT16)
    return NDArray.from_numpy(a.astype({FLOAT32: np.float32, DOUBLE: np.float64, HALF: np.float16}[dt]))


def _no_alloc(ex, op, X, n, stream=None):
    L = ex.L
    Z = NDArray.empty((), X.dtype)
    L.dbAllocateSpecialBuffer(Z.buffer.ptr)
    rc = L.nd4jhipReduceSameScalarNoAlloc(stream, op, X.dtype, L.dbSpecialBuffer(X.buffer.ptr), n, L.dbSpecialBuffer(Z.buffer.ptr))
    N.check("nd4jhipReduceSameScalarNoAlloc")
    assert rc == 0
    if stream:
        L.streamSynchronize(stream)
    L.dbTickDeviceWrite(Z.buffer.ptr)
    return Z.to_numpy()


@pytest.mark.parametrize("dt", [FLOAT32, DOUBLE, HALF, BFLOAT16])
@pytest.mark.parametrize("op", [ReduceSame.Sum, ReduceSame.Max, ReduceSame.Min, 3, 4, 5, 6])
def test_no_alloc_reduce_matches_exec_reduce_same(ex, dt, op):
    ex.L.initializeDevicesAndFunctions()
    rng = np.random.default_rng(100 * dt + op)
    scale = 1.0 if op != 3 else 1e-4                       # Prod: keep |x| near 1 so the product stays finite
    for n in (3_000_001, 70_001, 513):                     # split over many blocks, then fewer, then a single block
        a = rng.normal(0, 1, n) if op != 3 else 1.0 + scale * rng.normal(0, 1, n)
        X = _device(a, dt)
        X.sync_to_device()
        want = ex.exec_reduce_same(op, X, None).to_numpy()
        got = _no_alloc(ex, op, X, n)
        assert got.tobytes() == want.tobytes(), (n, got, want)


@pytest.mark.parametrize("dt", [FLOAT32, DOUBLE, HALF, BFLOAT16])
def test_no_alloc_reduce_of_short_arrays_allocates_nothing(ex, dt):
    """One element, and the lengths whose bytes select the 8-, 16- and 32-lanes-per-row launches; the device's free memory
    is the same before and after the calls."""
    L = ex.L
    L.initializeDevicesAndFunctions()
    rng = np.random.default_rng(dt)
    cases = []
    for n in (1, 7, 64, 200, 3000):
        X = _device(rng.normal(0, 1, n), dt)
        X.sync_to_device()
        Z = NDArray.empty((), dt)
        L.dbAllocateSpecialBuffer(Z.buffer.ptr)
        cases.append((n, X, Z, [ex.exec_reduce_same(op, X, None).to_numpy() for op in (ReduceSame.Sum, ReduceSame.Max, ReduceSame.AMin)]))
    ex.synchronize()
    free_before = L.getDeviceFreeMemory(L.getDevice())
    for n, X, Z, want in cases:
        for op, w in zip((ReduceSame.Sum, ReduceSame.Max, ReduceSame.AMin), want):
            assert L.nd4jhipReduceSameScalarNoAlloc(None, op, dt, L.dbSpecialBuffer(X.buffer.ptr), n, L.dbSpecialBuffer(Z.buffer.ptr)) == 0, L.lastErrorMessage()
            L.streamSynchronize(None)
            assert L.getDeviceFreeMemory(L.getDevice()) == free_before, ("the call changed the device's free memory", n, op)
            L.dbTickDeviceWrite(Z.buffer.ptr)
            got = Z.to_numpy()
            assert got.tobytes() == w.tobytes(), (n, op, got, w)


def test_no_alloc_reduce_on_a_caller_stream_and_limits(ex):
    L = ex.L
    L.initializeDevicesAndFunctions()
    x = np.random.default_rng(5).normal(0, 1, 1 << 20).astype(np.float32)
    X = NDArray.from_numpy(x)
    X.sync_to_device()
    want = ex.exec_reduce_same(ReduceSame.Sum, X, None).to_numpy()
    ex.synchronize()
    stream = L.createStream()
    got = _no_alloc(ex, ReduceSame.Sum, X, x.size, stream)
    assert got.tobytes() == want.tobytes()
    Z = NDArray.empty((), FLOAT32)
    L.dbAllocateSpecialBuffer(Z.buffer.ptr)
    for bad_n, msg in ((0, "at least 1"), (1 << 31, "exceeds the maximum")):
        assert L.nd4jhipReduceSameScalarNoAlloc(None, 0, FLOAT32, L.dbSpecialBuffer(X.buffer.ptr), bad_n, L.dbSpecialBuffer(Z.buffer.ptr)) == 1
        assert msg in L.lastErrorMessage().decode()
    assert L.nd4jhipReduceSameScalarNoAlloc(None, 0, 9, L.dbSpecialBuffer(X.buffer.ptr), 16, L.dbSpecialBuffer(Z.buffer.ptr)) == 1
    assert "FLOAT" in L.lastErrorMessage().decode()
