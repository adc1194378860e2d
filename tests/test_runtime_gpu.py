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


def test_recorded_copies_and_fills_replay_in_both_modes(ex, oracle):
    """memsetAsync and a device-to-device memcpyAsync issued on the library's stream between Begin and End belong to the
    recording: both replay modes must run them, also when the ops around them were merged (Add + layer_norm become one
    kernel, so the kept graph is the re-recorded plan).  Array handles and the OpContext are dropped before End."""
    import gc
    L = ex.L
    rng = np.random.default_rng(77)
    rows, cols = 8, 768
    gain, bias = rng.normal(1, 0.02, cols).astype(np.float32), rng.normal(0, 0.02, cols).astype(np.float32)
    X, Y = NDArray.empty((rows, cols), FLOAT32), NDArray.empty((rows, cols), FLOAT32)
    S, Ln, T, U = (NDArray.empty((rows, cols), FLOAT32) for _ in range(4))
    G, B = NDArray.from_numpy(gain), NDArray.from_numpy(bias)
    for a in (X, Y, S, Ln, T, U, G, B):
        a.sync_to_device()
    nbytes = rows * cols * 4
    dT, dU, dLn = (L.dbSpecialBuffer(a.buffer.ptr) for a in (T, U, Ln))

    def sequence(keep):
        # fill, add, normalise, copy the normalised rows out -- the handles used by the op calls die right after them
        assert L.memsetAsync(dU, 0, nbytes, 0, None) == 1
        x, y, s, ln = X.view(X.shape, X.strides), Y.view(Y.shape, Y.strides), S.view(S.shape, S.strides), Ln.view(Ln.shape, Ln.strides)
        L.execPairwiseTransform(None, Pairwise.Add, x.handle, y.handle, s.handle, None)
        N.check("execPairwiseTransform")
        call = ex.bind_custom("layer_norm", [s, G, B], [ln], i_args=[1], b_args=[False])
        call()
        assert L.memcpyAsync(dT, dLn, nbytes, 3, None) == 1
        if not keep:
            del call, x, y, s, ln
            gc.collect()

    def fresh(seed):
        r = np.random.default_rng(seed)
        x, y = r.normal(0, 1, (rows, cols)).astype(np.float32), r.normal(0, 1, (rows, cols)).astype(np.float32)
        X.assign_numpy(x); Y.assign_numpy(y)
        T.assign_numpy(np.full((rows, cols), -5.0, np.float32)); U.assign_numpy(np.ones((rows, cols), np.float32))
        for a in (T, U):
            a.sync_to_device()
        return x, y

    def read(a):
        L.dbTickDeviceWrite(a.buffer.ptr)     # the raw copy / fill wrote device memory behind the buffer's stamps
        return a.to_numpy()

    # eager
    x, y = fresh(1)
    sequence(keep=True)
    ex.synchronize()
    eager_ln = Ln.to_numpy()
    assert np.array_equal(read(T), eager_ln) and not read(U).any()
    assert_close(eager_ln, oracle.layer_norm(x + y, gain, bias, np.zeros_like(x), [1], channels_first=False), 1e-5, 1e-5, "eager")
    # recorded
    assert L.nd4jhipGraphBeginCapture() == 0, L.lastErrorMessage()
    sequence(keep=False)
    g = L.nd4jhipGraphEndCapture()
    N.check("nd4jhipGraphEndCapture")
    assert g and L.nd4jhipGraphFusedOps(g) == 1
    try:
        for i, mode in enumerate((0, 1, 0, 1)):
            L.nd4jhipSetGraphReplayMode(mode)
            x, y = fresh(10 + i)
            assert L.nd4jhipGraphLaunch(g) == 0, L.lastErrorMessage()
            ex.synchronize()
            want = oracle.layer_norm(x + y, gain, bias, np.zeros_like(x), [1], channels_first=False)
            got = Ln.to_numpy()
            assert_close(got, want, 1e-5, 1e-5, "replay %d" % i)
            assert np.array_equal(read(T), got), ("the recorded copy did not run", mode)
            assert not read(U).any(), ("the recorded fill did not run", mode)
    finally:
        L.nd4jhipSetGraphReplayMode(0)
        L.nd4jhipGraphDestroy(g)
    # a copy that touches host memory cannot be part of a recording
    host = L.mallocHost(64, 0)
    assert L.nd4jhipGraphBeginCapture() == 0
    assert L.memcpyAsync(host, dT, 64, 2, None) == 0
    assert b"device-to-device" in L.lastErrorMessage()
    g2 = L.nd4jhipGraphEndCapture()
    L.lastErrorMessage()
    if g2:
        L.nd4jhipGraphDestroy(g2)
    L.freeHost(host)
