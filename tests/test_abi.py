"""CPU tests of the C-ABI library: it loads, exports every declared entry point, and its host-side logic
(op hash, registry listing, descriptor cache, TAD packs, error slot) behaves like the reference's.
No compute entry point is called here."""
import ctypes
import os

import numpy as np
import pytest

from deeplearning4j_amd import nativeops as N

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    L = N.load()
    names = N.declared_symbols()
    assert len(names) > 120
    missing = [n for n in names if not hasattr(L, n)]
    assert not missing, missing
    untyped = [n for n in names if n not in N._SIGS and n not in ("setOmpNumThreads", "ompGetMaxThreads", "setElementThreshold", "setTADThreshold",
                                                                 "initializeShapeCache", "initializeTadCache", "deleteConstantShapeBuffer", "deleteTadPack")]
    assert not untyped, untyped


def test_op_hash_reference_vectors():
    # libnd4j/tests_cpu/layers_tests/HashUtilsTests.cpp:28-41
    L = N.load()
    assert L.nd4jhipOpHash(b"Conv2D") == -1637140380760460323
    assert L.nd4jhipOpHash(b"switch") == -1988317239813741487


def test_registry_listing_format(oracle):
    L = N.load()
    items = [i for i in L.getAllCustomOps().decode().split(";") if i]
    names = {}
    for it in items:
        parts = it.split(":")
        assert len(parts) == 8 and parts[7] == ""       # name:hash:nIn:nOut:inplace:nT:nI:
        names[parts[0]] = int(parts[1])
        assert int(parts[1]) == oracle.hash_name(parts[0])
    for op in ("matmul", "mmul", "mMul", "gemm", "softmax", "layer_norm", "dot_product_attention_v2", "argmax", "argmin"):
        assert op in names


def _si(L, shape, strides, dtype=5, order=b"c"):
    sh = (ctypes.c_longlong * max(len(shape), 1))(*shape)
    st = (ctypes.c_longlong * max(len(strides), 1))(*strides) if strides is not None else None
    buf = L.shapeBuffer(len(shape), sh, st, dtype, order, 1, False)
    p = ctypes.cast(L.getConstantShapeBufferPrimary(buf), ctypes.POINTER(ctypes.c_longlong))
    n = 6 if len(shape) == 0 else 2 * len(shape) + 4
    return buf, [p[i] for i in range(n)]


def test_shape_buffer_layout():
    L = N.load()
    # config-1 descriptor: [2, 8192, 4096, 4096, 1, 8192, 1, 99]
    _, si = _si(L, [8192, 4096], None)
    assert si == [2, 8192, 4096, 4096, 1, 8192, 1, 99]
    _, si = _si(L, [3, 4], None, 17, b"f")
    assert si == [2, 3, 4, 1, 3, 2048, 1, 102]
    _, si = _si(L, [], None, 10)
    assert si == [0, 0, 1, 262144, 1, 99]
    b1, si = _si(L, [2, 3], [1, 2], 6)
    assert si == [2, 2, 3, 1, 2, 16384, 0, 99]
    b2, _ = _si(L, [2, 3], [1, 2], 6)
    assert b1 == b2                                      # cached: same descriptor, same buffer


def test_tad_pack_matches_oracle(oracle):
    L = N.load()
    from deeplearning4j_amd.ndarray import DataBuffer, INT64, make_shape_info
    for shape, dims in [((5, 5), [1]), ((2, 3, 4), [0, 2]), ((2, 3, 4, 5), [1, 3]), ((3, 4), [0, 1])]:
        a = np.zeros(shape, np.float32)
        si = make_shape_info(shape, [s // 4 for s in a.strides], 5)
        buf = DataBuffer(len(si), INT64, allocate_both=False)
        buf.host_view()[: len(si)] = si
        d = (ctypes.c_longlong * len(dims))(*dims)
        pack = L.tadOnlyShapeInfo(buf.ptr, d, len(dims))
        N.check("tadOnlyShapeInfo")
        n = L.getNumberOfTads(pack)
        tsi_want, offs_want = oracle.tad(a, dims)
        assert n == len(offs_want)
        offs = L.getPrimaryOffsets(pack)
        assert [offs[i] for i in range(n)] == list(offs_want)
        tsi = L.getPrimaryShapeInfo(pack)
        ln = L.getShapeInfoLength(pack)
        assert ln == len(tsi_want)
        got = [tsi[i] for i in range(ln)]
        rank = got[0]
        assert got[:1 + 2 * rank] == list(tsi_want[:1 + 2 * rank])


def test_error_slot_semantics():
    # a failure parks {code, message}; fetching the message consumes the code (execution/impl/ErrorReference.cpp:28-34)
    L = N.load()
    L.lastErrorMessage()
    assert L.lastErrorCode() == 0
    assert L.createOpaqueNDArray(None, None, None, 0) is None
    assert L.lastErrorCode() == 1
    assert L.lastErrorCode() == 1
    assert b"Shape info was null" in L.lastErrorMessage()
    assert L.lastErrorCode() == 0
    # unknown op hash -> non-zero status + message
    ctx = L.createGraphContext(1)
    assert L.execCustomOp2(None, 12345, ctx) != 0
    assert b"unknown op hash" in L.lastErrorMessage()
    L.deleteGraphContext(ctx)
    # null operands on a legacy loop
    L.execReduceFloat(None, 0, None, None, None)
    assert L.lastErrorCode() == 1
    assert b"null pointer" in L.lastErrorMessage()


def test_context_argument_round_trip():
    L = N.load()
    ctx = L.createGraphContext(7)
    L.setGraphContextTArguments(ctx, (ctypes.c_double * 2)(0.125, 0.0), 2)
    L.setGraphContextIArguments(ctx, (ctypes.c_longlong * 3)(0, 1, -1), 3)
    L.setGraphContextBArguments(ctx, (ctypes.c_bool * 2)(True, False), 2)
    L.setGraphContextDArguments(ctx, (ctypes.c_int * 1)(10), 1)
    assert (L.numTArgumentsNative(ctx), L.numIArgumentsNative(ctx), L.numBNative(ctx), L.numDNative(ctx)) == (2, 3, 2, 1)
    assert L.tArgumentNative(ctx, 0) == 0.125 and L.iArgumentAtNative(ctx, 2) == -1 and L.bArgAtNative(ctx, 0) and L.dataTypeNativeAt(ctx, 0) == 10
    assert L.numInputsNative(ctx) == 0 and L.getInputArrayNative(ctx, 0) is None
    L.ctxPurge(ctx)
    assert L.numIArgumentsNative(ctx) == 0
    L.deleteGraphContext(ctx)


def test_compute_without_gpu_fails_loudly():
    L = N.load()
    if L.getAvailableDevices() > 0:
        pytest.skip("a GPU is present")
    L.initializeDevicesAndFunctions()
    assert L.lastErrorCode() != 0
    assert b"no CPU fallback" in L.lastErrorMessage()


def test_start_up_queries_and_out_of_scope_entry_points():
    # what a device backend asks while it starts (AtomicAllocator.java:140 enableP2P, CudaAffinityManager.java:353
    # isP2PAvailable, the executioner's version and capability checks): answered without a device
    L = N.load()
    L.lastErrorMessage()
    assert L.isBlasVersionMatches(12, 3, 0) is True        # no vendor BLAS underneath, nothing to mismatch
    assert (L.binaryLevel(), L.optimalLevel()) == (0, 0)   # legacy/cuda/NativeOps.cu:2769-2775
    assert L.isMinimalRequirementsMet() and L.isOptimalRequirementsMet() and not L.isExperimentalEnabled()
    L.initializeFunctions(None); L.setOmpMinThreads(4); L.setGridLimit(128)
    assert L.getConstantSpace() is None and L.lcSolverHandle(None) is None and L.lcBlasHandlePtr(None) is None
    L.checkP2P()
    # fewer than two devices: the reference reports peer access as available (legacy/cuda/NativeOps.cu:1046-1049)
    if L.getAvailableDevices() < 2:
        assert L.isP2PAvailable() is True
    L.enableP2P(True); L.enableP2P(False)
    assert L.lastErrorCode() == 0
    # the by-pointer overloads read the handle through the pointer
    null_handle = ctypes.c_void_p(None)
    assert L.lcExecutionStreamPtr(ctypes.byref(null_handle)) is None and L.lcScalarPointerPtr(None) is None
    # entry points outside this backend's path resolve, do nothing and say so in the error slot
    for name, args in (("execRandom", (None, 0, None, None, None)), ("execRandom2", (None, 0, None, None, None, None)),
                       ("execRandom3", (None, 0, None, None, None, None, None)), ("sort", (None, None, False)),
                       ("sortTad", (None, None, None, 0, None, None, False)), ("shuffle", (None, None, None, 0, None, None)),
                       ("pullRows", (None, None, None, 0, None, 0)), ("convertTypes", (None, 5, None, 0, 6, None))):
        getattr(L, name)(*args)
        assert L.lastErrorCode() == 1
        assert (name + " is not implemented in nd4j-hip").encode() in L.lastErrorMessage()


def test_profiler_detection_keeps_graph_launches_off_the_tracer():
    # nd4jhipGraphLaunch replays kernel by kernel when a rocprofiler tool library is attached; the detection reads the
    # environment the tool is started with and the list of loaded objects.  Each case in a fresh process.
    import subprocess
    import sys
    code = ("import sys; sys.path.insert(0, %r); from deeplearning4j_amd import nativeops as N; "
            "print(N.load().nd4jhipProfilerAttached())" % ROOT)
    def run(extra):
        env = {k: v for k, v in os.environ.items() if k not in ("ROCP_TOOL_LIBRARIES",)}
        env.update(extra)
        return subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=120).stdout.strip().splitlines()[-1]
    assert run({}) == "0"
    assert run({"ROCP_TOOL_LIBRARIES": "/opt/rocm/lib/rocprofiler-sdk/librocprofiler-sdk-tool.so"}) == "1"


def test_attention_block_order_is_a_balanced_permutation():
    """The host-side table that deals the query tiles of a causal attention launch out over the block ids: every item
    once, the block ids that share a CU (id mod 256) within a few key tiles of each other, and with a multiple of 8 batch
    entries every batch entry on one XCD (id mod 8)."""
    import ctypes
    L = N.load()
    def order(nb, qt, per, resident):
        buf = (ctypes.c_ushort * max(nb * qt, 1))()
        n = L.nd4jhipAttentionBlockOrder(nb, qt, per, resident, buf)
        return list(buf[:n])
    for nb, qt, per, resident, by_xcd in ((96, 8, 2, 3, True), (96, 8, 4, 3, True), (40, 8, 2, 3, True), (50, 6, 2, 3, False), (37, 10, 2, 3, False),
                                          (64, 8, 2, 2, True)):
        items = order(nb, qt, per, resident)
        total = nb * qt
        assert sorted(items) == list(range(total)), (nb, qt)
        load = [0] * 256
        for block, item in enumerate(items):
            slot, b = divmod(item, nb)
            load[block % 256] += per * (qt - slot) + 1
            if by_xcd:
                assert block % 8 == b % 8, (nb, qt, block, item)
        used = [v for v in load if v]
        mean = sum(load) / 256.0
        heaviest = per * qt + 1
        # no CU more than one light tile above an even share (or above the heaviest single tile, when that is more)
        assert max(load) <= max(mean, heaviest) + 2 * per + 2, (nb, qt, max(load), mean)
        assert len(used) == min(total, 256)
    # launches that are not on the chip at once, or have at most a block per CU, keep the plain order
    assert order(96, 8, 2, 2) == [] and order(2, 8, 2, 3) == [] and order(200, 8, 2, 3) == [] and order(96, 1, 2, 3) == []

