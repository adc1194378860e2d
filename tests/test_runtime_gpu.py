"""Boundary behaviour that needs a device: two caller threads, a caller-owned stream, stamps across graph replays."""
import ctypes
import math
import threading

import numpy as np
import pytest

from conftest import assert_close
from deeplearning4j_amd import nativeops as N
from deeplearning4j_amd.executioner import Pairwise, ReduceSame
from deeplearning4j_amd.ndarray import BFLOAT16, FLOAT32, NDArray, bf16_bits_to_f32, f32_to_bf16_bits

pytestmark = pytest.mark.gpu


def test_two_caller_threads_do_not_mix_scratch(ex):
    """Split-K matmuls park partial tiles in the library's scratch and full reductions park block partials there; two
    threads issuing them at once (ctypes releases the GIL during a native call) must each get their own result."""
    rng = np.random.default_rng(11)
    M, K, Nn = 32, 3072, 768
    work = []
    for t in range(2):
        a = f32_to_bf16_bits(rng.normal(0, 1 / math.sqrt(K), (M, K)).astype(np.float32))
        b = f32_to_bf16_bits(rng.normal(0, 1, (K, Nn)).astype(np.float32))
        x = rng.normal(0, 1, (1 << 22,)).astype(np.float32)
        A, B, X = NDArray.from_numpy(a, BFLOAT16), NDArray.from_numpy(b, BFLOAT16), NDArray.from_numpy(x)
        want_mm = ex.exec_custom("matmul", [A, B])[0].to_numpy()
        assert "splitk" in ex.L.nd4jhipLastGemmKernel().decode()
        want_sum = ex.exec_reduce_same(ReduceSame.Sum, X, None).to_numpy()
        assert_close(bf16_bits_to_f32(want_mm), bf16_bits_to_f32(a).astype(np.float64) @ bf16_bits_to_f32(b).astype(np.float64), 1e-2, 1e-2, "matmul")
        work.append((A, B, X, want_mm, want_sum))
    errors = []

    def run(t):
        A, B, X, want_mm, want_sum = work[t]
        try:
            for _ in range(150):
                got = ex.exec_custom("matmul", [A, B])[0].to_numpy()
                if not np.array_equal(got, want_mm):
                    errors.append("thread %d: matmul result changed" % t)
                    return
                got = ex.exec_reduce_same(ReduceSame.Sum, X, None).to_numpy()
                if not np.array_equal(got, want_sum):
                    errors.append("thread %d: reduction result changed" % t)
                    return
        except Exception as e:   # noqa: BLE001
            errors.append("thread %d: %r" % (t, e))

    threads = [threading.Thread(target=run, args=(t,)) for t in range(2)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    assert not errors, errors


def test_caller_stream_is_ordered_before_the_op(ex):
    """A device backend queues its own copies on its stream and passes that stream with the op (extraPointers[1] for the
    legacy loops, setGraphContextCudaContext for declarable ops): the op must see the copied data."""
    L = ex.L
    n = 1 << 25                                   # 128 MiB: the copy is still in flight when the op call arrives
    nbytes = n * 4
    stream = L.createStream()
    N.check("createStream")
    host = L.mallocHost(nbytes, 0)
    N.check("mallocHost")
    src = np.frombuffer((ctypes.c_char * nbytes).from_address(host), dtype=np.float32, count=n)
    X = NDArray.empty((n,), FLOAT32)
    Y = NDArray.from_numpy(np.ones(n, np.float32))
    Y.sync_to_device()
    Z = NDArray.empty((n,), FLOAT32)
    L.dbAllocateSpecialBuffer(X.buffer.ptr)
    extra = (ctypes.c_void_p * 16)()
    extra[1] = stream
    for round_ in range(3):
        src[:] = float(round_ + 1)
        assert L.memcpyAsync(L.dbSpecialBuffer(X.buffer.ptr), host, nbytes, 1, stream) == 1
        L.dbTickDeviceWrite(X.buffer.ptr)
        L.execPairwiseTransform(extra, Pairwise.Add, X.handle, Y.handle, Z.handle, None)
        N.check("execPairwiseTransform")
        got = Z.to_numpy()
        assert got[0] == round_ + 2 and got[-1] == round_ + 2 and np.all(got == round_ + 2)
    # the same through an op context
    src[:] = 7.0
    assert L.memcpyAsync(L.dbSpecialBuffer(X.buffer.ptr), host, nbytes, 1, stream) == 1
    L.dbTickDeviceWrite(X.buffer.ptr)
    ctx = L.createGraphContext(1)
    L.setGraphContextCudaContext(ctx, stream, None, None)
    ins = (ctypes.c_void_p * 2)(X.handle, Y.handle)
    outs = (ctypes.c_void_p * 1)(Z.handle)
    L.setGraphContextInputArraysArr(ctx, 2, ins)
    L.setGraphContextOutputArraysArr(ctx, 1, outs)
    assert L.execCustomOp2(None, L.nd4jhipOpHash(b"add"), ctx) == 0, L.lastErrorMessage()
    assert np.all(Z.to_numpy() == 8.0)
    L.deleteGraphContext(ctx)
    L.streamSynchronize(stream)
    L.freeHost(host)


@pytest.mark.parametrize("replay_mode", [0, 1])
def test_graph_replay_keeps_buffer_stamps(ex, replay_mode):
    """A replayed graph must upload an input the host rewrote after the capture and must mark what it writes, so that a
    host read after each replay returns that replay's values (not the copy fetched after the previous one).  Both ways
    of replaying (the graph; the recorded sequence launched kernel by kernel)."""
    ex.L.nd4jhipSetGraphReplayMode(replay_mode)
    try:
        _graph_replay_keeps_buffer_stamps(ex)
    finally:
        ex.L.nd4jhipSetGraphReplayMode(0)


def test_recording_outlives_the_callers_array_handles(ex):
    """A recording holds its own views of the arrays it was made on: the caller may drop its view handles (the buffers
    stay), and both ways of replaying still write the right columns."""
    import gc
    L = ex.L
    rng = np.random.default_rng(77)
    a, b = rng.normal(0, 1, (64, 96)).astype(np.float32), rng.normal(0, 1, (64, 96)).astype(np.float32)
    A, B, Z = NDArray.from_numpy(a), NDArray.from_numpy(b), NDArray.from_numpy(np.zeros((64, 96), np.float32))
    for arr in (A, B, Z):
        arr.sync_to_device()
    va, vb, vz = A.slice(1, 8, 72), B.slice(1, 16, 80), Z.slice(1, 32, 96)
    assert L.nd4jhipGraphBeginCapture() == 0, L.lastErrorMessage()
    L.execPairwiseTransform(None, Pairwise.Add, va.handle, vb.handle, vz.handle, None)
    g = L.nd4jhipGraphEndCapture()
    N.check("nd4jhipGraphEndCapture")
    assert g
    del va, vb, vz
    gc.collect()
    junk = [NDArray.from_numpy(np.full((64, 96), 7.0, np.float32)).slice(1, 1, 5) for _ in range(32)]   # recycles freed handles
    want = np.zeros((64, 96), np.float32)
    want[:, 32:] = a[:, 8:72] + b[:, 16:80]
    try:
        for mode in (1, 0, 1):
            L.nd4jhipSetGraphReplayMode(mode)
            Z.assign_numpy(np.zeros((64, 96), np.float32))
            assert L.nd4jhipGraphLaunch(g) == 0, L.lastErrorMessage()
            assert np.array_equal(Z.to_numpy(), want), mode
    finally:
        L.nd4jhipSetGraphReplayMode(0)
        L.nd4jhipGraphDestroy(g)
    assert len(junk) == 32


def _graph_replay_keeps_buffer_stamps(ex):
    L = ex.L
    x = np.arange(4096, dtype=np.float32)
    X, Y, Z = NDArray.from_numpy(x), NDArray.from_numpy(np.ones(4096, np.float32)), NDArray.empty((4096,), FLOAT32)
    X.sync_to_device(); Y.sync_to_device()
    L.dbAllocateSpecialBuffer(Z.buffer.ptr)
    assert L.nd4jhipGraphBeginCapture() == 0, L.lastErrorMessage()
    L.execPairwiseTransform(None, Pairwise.Add, X.handle, Y.handle, Z.handle, None)
    g = L.nd4jhipGraphEndCapture()
    N.check("nd4jhipGraphEndCapture")
    assert g
    assert L.nd4jhipGraphLaunch(g) == 0, L.lastErrorMessage()
    assert np.array_equal(Z.to_numpy(), x + 1)
    for k in (2.0, 3.0):
        X.assign_numpy(x * k)                       # host write after the capture
        assert L.nd4jhipGraphLaunch(g) == 0, L.lastErrorMessage()
        assert np.array_equal(Z.to_numpy(), x * k + 1)
    L.nd4jhipGraphDestroy(g)
