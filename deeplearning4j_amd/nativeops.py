"""ctypes binding of libnd4jhip.so -- the stand-in for the JavaCPP-generated `Nd4jHip` class.

Mirrors the Java interface `org.nd4j.nativeblas.NativeOps`
(nd4j/nd4j-backends/nd4j-api-parent/nd4j-api/src/main/java/org/nd4j/nativeblas/NativeOps.java)
for the functions on the op path: same names, same argument order.  Signatures are taken from
include/nd4jhip/NativeOps.h.

There is no CPU fallback: if the library is missing, loading fails; if no GPU is present, compute
calls set the error slot, which `check()` turns into an exception.
"""
import ctypes
import os
import re

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libnd4jhip.so")
HEADER_PATH = os.path.join(os.path.dirname(HERE), "include", "nd4jhip", "NativeOps.h")

c_long = ctypes.c_longlong
c_ptr = ctypes.c_void_p
LongPtr = ctypes.POINTER(ctypes.c_longlong)


class NativeOpsError(RuntimeError):
    pass


_SIGS = {
    # name: (restype, argtypes)
    "initializeDevicesAndFunctions": (None, []),
    "getAvailableDevices": (ctypes.c_int, []),
    "setDevice": (ctypes.c_int, [ctypes.c_int]),
    "getDevice": (ctypes.c_int, []),
    "getDeviceName": (ctypes.c_char_p, [ctypes.c_int]),
    "getDeviceMajor": (ctypes.c_int, [ctypes.c_int]),
    "getDeviceMinor": (ctypes.c_int, [ctypes.c_int]),
    "getDeviceFreeMemory": (c_long, [ctypes.c_int]),
    "getDeviceFreeMemoryDefault": (c_long, []),
    "getDeviceTotalMemory": (c_long, [ctypes.c_int]),
    "enableDebugMode": (None, [ctypes.c_bool]),
    "enableVerboseMode": (None, [ctypes.c_bool]),
    "lastErrorCode": (ctypes.c_int, []),
    "lastErrorMessage": (ctypes.c_char_p, []),
    "mallocHost": (c_ptr, [c_long, ctypes.c_int]),
    "mallocDevice": (c_ptr, [c_long, ctypes.c_int, ctypes.c_int]),
    "freeHost": (ctypes.c_int, [c_ptr]),
    "freeDevice": (ctypes.c_int, [c_ptr, ctypes.c_int]),
    "createStream": (c_ptr, []),
    "createEvent": (c_ptr, []),
    "registerEvent": (ctypes.c_int, [c_ptr, c_ptr]),
    "destroyEvent": (ctypes.c_int, [c_ptr]),
    "streamSynchronize": (ctypes.c_int, [c_ptr]),
    "eventSynchronize": (ctypes.c_int, [c_ptr]),
    "memcpySync": (ctypes.c_int, [c_ptr, c_ptr, c_long, ctypes.c_int, c_ptr]),
    "memcpyAsync": (ctypes.c_int, [c_ptr, c_ptr, c_long, ctypes.c_int, c_ptr]),
    "memsetSync": (ctypes.c_int, [c_ptr, ctypes.c_int, c_long, ctypes.c_int, c_ptr]),
    "memsetAsync": (ctypes.c_int, [c_ptr, ctypes.c_int, c_long, ctypes.c_int, c_ptr]),
    "defaultLaunchContext": (c_ptr, []),
    "lcScalarPointer": (c_ptr, [c_ptr]),
    "lcReductionPointer": (c_ptr, [c_ptr]),
    "lcAllocationPointer": (c_ptr, [c_ptr]),
    "lcExecutionStream": (c_ptr, [c_ptr]),
    "lcCopyStream": (c_ptr, [c_ptr]),
    "lcBlasHandle": (c_ptr, [c_ptr]),
    "dbAllocateDataBuffer": (c_ptr, [c_long, ctypes.c_int, ctypes.c_bool]),
    "allocateDataBuffer": (c_ptr, [c_long, ctypes.c_int, ctypes.c_bool]),
    "dbCreateExternalDataBuffer": (c_ptr, [c_long, ctypes.c_int, c_ptr, c_ptr]),
    "dbCreateView": (c_ptr, [c_ptr, c_long]),
    "dbPrimaryBuffer": (c_ptr, [c_ptr]),
    "dbSpecialBuffer": (c_ptr, [c_ptr]),
    "dbBufferLength": (c_long, [c_ptr]),
    "dbSetPrimaryBuffer": (None, [c_ptr, c_ptr, c_long]),
    "dbSetSpecialBuffer": (None, [c_ptr, c_ptr, c_long]),
    "dbAllocatePrimaryBuffer": (None, [c_ptr]),
    "dbAllocateSpecialBuffer": (None, [c_ptr]),
    "dbExpandBuffer": (None, [c_ptr, c_long]),
    "dbExpand": (None, [c_ptr, c_long]),
    "dbUseCount": (ctypes.c_int, [c_ptr]),
    "dbSyncToSpecial": (None, [c_ptr]),
    "dbSyncToPrimary": (None, [c_ptr]),
    "dbTickHostRead": (None, [c_ptr]),
    "dbTickHostWrite": (None, [c_ptr]),
    "dbTickDeviceRead": (None, [c_ptr]),
    "dbTickDeviceWrite": (None, [c_ptr]),
    "dbClose": (None, [c_ptr]),
    "dbDeviceId": (ctypes.c_int, [c_ptr]),
    "dbSetDeviceId": (None, [c_ptr, ctypes.c_int]),
    "dbLocality": (ctypes.c_int, [c_ptr]),
    "deleteDataBuffer": (None, [c_ptr]),
    "shapeBuffer": (c_ptr, [ctypes.c_int, LongPtr, LongPtr, ctypes.c_int, ctypes.c_char, c_long, ctypes.c_bool]),
    "shapeBufferEx": (c_ptr, [ctypes.c_int, LongPtr, LongPtr, ctypes.c_int, ctypes.c_char, c_long, c_long]),
    "cacheAndStoreShapeBuffer": (c_ptr, [LongPtr]),
    "getConstantShapeBufferPrimary": (c_ptr, [c_ptr]),
    "getConstantShapeBufferSpecial": (c_ptr, [c_ptr]),
    "createOpaqueNDArray": (c_ptr, [c_ptr, c_ptr, c_ptr, c_long]),
    "deleteNDArray": (None, [c_ptr]),
    "getOpaqueNDArrayOffset": (c_long, [c_ptr]),
    "getOpaqueNDArrayShapeInfo": (LongPtr, [c_ptr]),
    "getOpaqueNDArrayBuffer": (c_ptr, [c_ptr]),
    "getOpaqueNDArraySpecialBuffer": (c_ptr, [c_ptr]),
    "getOpaqueNDArrayLength": (c_long, [c_ptr]),
    "getOpaqueNDArrayShapeInfoLength": (c_long, [c_ptr]),
    "tadOnlyShapeInfo": (c_ptr, [c_ptr, LongPtr, c_long]),
    "getPrimaryShapeInfo": (LongPtr, [c_ptr]),
    "getPrimaryOffsets": (LongPtr, [c_ptr]),
    "getSpecialShapeInfo": (LongPtr, [c_ptr]),
    "getSpecialOffsets": (LongPtr, [c_ptr]),
    "getNumberOfTads": (c_long, [c_ptr]),
    "getShapeInfoLength": (ctypes.c_int, [c_ptr]),
    "execPairwiseTransform": (None, [c_ptr, ctypes.c_int, c_ptr, c_ptr, c_ptr, c_ptr]),
    "execTransformStrict": (None, [c_ptr, ctypes.c_int, c_ptr, c_ptr, c_ptr]),
    "execTransformFloat": (None, [c_ptr, ctypes.c_int, c_ptr, c_ptr, c_ptr]),
    "execTransformSame": (None, [c_ptr, ctypes.c_int, c_ptr, c_ptr, c_ptr]),
    "execTransformAny": (None, [c_ptr, ctypes.c_int, c_ptr, c_ptr, c_ptr]),
    "execReduceFloat": (None, [c_ptr, ctypes.c_int, c_ptr, c_ptr, c_ptr]),
    "execReduceFloat2": (None, [c_ptr, ctypes.c_int, c_ptr, c_ptr, c_ptr, c_ptr]),
    "execReduceSame": (None, [c_ptr, ctypes.c_int, c_ptr, c_ptr, c_ptr]),
    "execReduceSame2": (None, [c_ptr, ctypes.c_int, c_ptr, c_ptr, c_ptr, c_ptr]),
    "execIndexReduce": (None, [c_ptr, ctypes.c_int, c_ptr, c_ptr, c_ptr, c_ptr]),
    "execIndexReduceScalar": (None, [c_ptr, ctypes.c_int, c_ptr, c_ptr, c_ptr]),
    "execTransformBool": (None, [c_ptr, ctypes.c_int, c_ptr, c_ptr, c_ptr]),
    "execSummaryStatsScalar": (None, [c_ptr, ctypes.c_int, c_ptr, c_ptr, c_ptr, ctypes.c_bool]),
    "execSummaryStatsTad": (None, [c_ptr, ctypes.c_int, c_ptr, c_ptr, c_ptr, c_ptr, ctypes.c_bool]),
    "execReduce3": (None, [c_ptr, ctypes.c_int, c_ptr, c_ptr, c_ptr, c_ptr]),
    "execReduce3Scalar": (None, [c_ptr, ctypes.c_int, c_ptr, c_ptr, c_ptr, c_ptr]),
    "execReduce3Tad": (None, [c_ptr, ctypes.c_int, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr]),
    "execReduce3All": (None, [c_ptr, ctypes.c_int, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr]),
    "execReduceLong": (None, [c_ptr, ctypes.c_int, c_ptr, c_ptr, c_ptr, c_ptr]),
    "execReduceLong2": (None, [c_ptr, ctypes.c_int, c_ptr, c_ptr, c_ptr, c_ptr]),
    "execReduceBool": (None, [c_ptr, ctypes.c_int, c_ptr, c_ptr, c_ptr, c_ptr]),
    "execReduceBool2": (None, [c_ptr, ctypes.c_int, c_ptr, c_ptr, c_ptr, c_ptr]),
    "execScalar": (None, [c_ptr, ctypes.c_int, c_ptr, c_ptr, c_ptr, c_ptr]),
    "execBroadcast": (None, [c_ptr, ctypes.c_int, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr]),
    "execPairwiseTransformBool": (None, [c_ptr, ctypes.c_int, c_ptr, c_ptr, c_ptr, c_ptr]),
    "execBroadcastBool": (None, [c_ptr, ctypes.c_int, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr]),
    "execScalarBool": (None, [c_ptr, ctypes.c_int, c_ptr, c_ptr, c_ptr, c_ptr]),
    "execScalarBoolTad": (None, [c_ptr, ctypes.c_int, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr]),
    "execScalarTad": (None, [c_ptr, ctypes.c_int, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr]),
    "getAllCustomOps": (ctypes.c_char_p, []),
    "createGraphContext": (c_ptr, [ctypes.c_int]),
    "deleteGraphContext": (None, [c_ptr]),
    "markGraphContextInplace": (None, [c_ptr, ctypes.c_bool]),
    "setGraphContextInputArray": (None, [c_ptr, ctypes.c_int, c_ptr]),
    "setGraphContextOutputArray": (None, [c_ptr, ctypes.c_int, c_ptr]),
    "setGraphContextInputArraysArr": (None, [c_ptr, ctypes.c_int, ctypes.POINTER(c_ptr)]),
    "setGraphContextOutputArraysArr": (None, [c_ptr, ctypes.c_int, ctypes.POINTER(c_ptr)]),
    "setGraphContextTArguments": (None, [c_ptr, ctypes.POINTER(ctypes.c_double), ctypes.c_int]),
    "setGraphContextIArguments": (None, [c_ptr, LongPtr, ctypes.c_int]),
    "setGraphContextBArguments": (None, [c_ptr, ctypes.POINTER(ctypes.c_bool), ctypes.c_int]),
    "setGraphContextDArguments": (None, [c_ptr, ctypes.POINTER(ctypes.c_int), ctypes.c_int]),
    "ctxAllowHelpers": (None, [c_ptr, ctypes.c_bool]),
    "ctxShapeFunctionOverride": (None, [c_ptr, ctypes.c_bool]),
    "ctxSetExecutionMode": (None, [c_ptr, ctypes.c_int]),
    "ctxPurge": (None, [c_ptr]),
    "getInputArrayNative": (c_ptr, [c_ptr, ctypes.c_int]),
    "getOutputArrayNative": (c_ptr, [c_ptr, ctypes.c_int]),
    "numInputsNative": (c_long, [c_ptr]),
    "numOutputsNative": (c_long, [c_ptr]),
    "numTArgumentsNative": (c_long, [c_ptr]),
    "numIArgumentsNative": (c_long, [c_ptr]),
    "numBNative": (c_long, [c_ptr]),
    "numDNative": (c_long, [c_ptr]),
    "tArgumentNative": (ctypes.c_double, [c_ptr, ctypes.c_int]),
    "iArgumentAtNative": (c_long, [c_ptr, ctypes.c_int]),
    "bArgAtNative": (ctypes.c_bool, [c_ptr, ctypes.c_int]),
    "dataTypeNativeAt": (c_long, [c_ptr, ctypes.c_int]),
    "execCustomOp2": (ctypes.c_int, [c_ptr, c_long, c_ptr]),
    "calculateOutputShapes2": (c_ptr, [c_ptr, c_long, c_ptr]),
    "getShapeListSize": (c_long, [c_ptr]),
    "getShape": (LongPtr, [c_ptr, c_long]),
    "deleteShapeList": (None, [c_ptr]),
    "nd4jhipOpHash": (c_long, [ctypes.c_char_p]),
    "nd4jhipCreateTimingEvent": (c_ptr, []),
    "nd4jhipEventElapsedMs": (ctypes.c_float, [c_ptr, c_ptr]),
    "nd4jhipSetSyncAfterCustomOp": (None, [ctypes.c_int]),
    "nd4jhipGraphBeginCapture": (ctypes.c_int, []),
    "nd4jhipGraphEndCapture": (c_ptr, []),
    "nd4jhipGraphLaunch": (ctypes.c_int, [c_ptr]),
    "nd4jhipGraphDestroy": (None, [c_ptr]),
    "nd4jhipGraphFusedOps": (ctypes.c_int, [c_ptr]),
    "nd4jhipGraphFusedApplied": (ctypes.c_int, [c_ptr]),
    "nd4jhipSetGraphReplayMode": (None, [ctypes.c_int]),
    "nd4jhipGetGraphReplayMode": (ctypes.c_int, []),
    "nd4jhipBuildInfo": (ctypes.c_char_p, []),
    "nd4jhipLastGemmKernel": (ctypes.c_char_p, []),
    "nd4jhipAttentionBlockOrder": (ctypes.c_int, [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.POINTER(ctypes.c_ushort)]),
    "nd4jhipReduceSameScalarNoAlloc": (ctypes.c_int, [c_ptr, ctypes.c_int, ctypes.c_int, c_ptr, c_long, c_ptr]),
    "setGraphContextCudaContext": (None, [c_ptr, c_ptr, c_ptr, c_ptr]),
    "nd4jhipProfilerAttached": (ctypes.c_int, []),
    "nd4jhipGraphAudit": (ctypes.c_int, [c_ptr]),
    "lcSolverHandle": (c_ptr, [c_ptr]),
    "lcScalarPointerPtr": (c_ptr, [ctypes.POINTER(c_ptr)]),
    "lcReductionPointerPtr": (c_ptr, [ctypes.POINTER(c_ptr)]),
    "lcAllocationPointerPtr": (c_ptr, [ctypes.POINTER(c_ptr)]),
    "lcExecutionStreamPtr": (c_ptr, [ctypes.POINTER(c_ptr)]),
    "lcCopyStreamPtr": (c_ptr, [ctypes.POINTER(c_ptr)]),
    "lcBlasHandlePtr": (c_ptr, [ctypes.POINTER(c_ptr)]),
    "checkP2P": (None, []),
    "enableP2P": (None, [ctypes.c_bool]),
    "isP2PAvailable": (ctypes.c_bool, []),
    "initializeFunctions": (None, [ctypes.POINTER(c_ptr)]),
    "isBlasVersionMatches": (ctypes.c_bool, [ctypes.c_int, ctypes.c_int, ctypes.c_int]),
    "binaryLevel": (ctypes.c_int, []),
    "optimalLevel": (ctypes.c_int, []),
    "isMinimalRequirementsMet": (ctypes.c_bool, []),
    "isOptimalRequirementsMet": (ctypes.c_bool, []),
    "isExperimentalEnabled": (ctypes.c_bool, []),
    "setOmpMinThreads": (None, [ctypes.c_int]),
    "setGridLimit": (None, [ctypes.c_int]),
    "getConstantSpace": (c_ptr, []),
    "execRandom": (None, [c_ptr, ctypes.c_int, c_ptr, c_ptr, c_ptr]),
    "execRandom2": (None, [c_ptr, ctypes.c_int, c_ptr, c_ptr, c_ptr, c_ptr]),
    "execRandom3": (None, [c_ptr, ctypes.c_int, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr]),
    "sort": (None, [c_ptr, c_ptr, ctypes.c_bool]),
    "sortTad": (None, [c_ptr, c_ptr, LongPtr, c_long, LongPtr, LongPtr, ctypes.c_bool]),
    "shuffle": (None, [c_ptr, c_ptr, c_ptr, ctypes.c_int, c_ptr, c_ptr]),
    "pullRows": (None, [c_ptr, c_ptr, c_ptr, c_long, c_ptr, c_long]),
    "convertTypes": (None, [c_ptr, ctypes.c_int, c_ptr, c_long, ctypes.c_int, c_ptr]),
}


def declared_symbols():
    """Every entry point include/nd4jhip/NativeOps.h declares."""
    text = open(HEADER_PATH).read()
    text = text.replace("#define ND4JHIP_EXPORT", "#define _EXPORT_MACRO")
    return re.findall(r"ND4JHIP_EXPORT\s+[^;(]*?\b(\w+)\s*\(", text)


_lib = None


def load():
    """Load libnd4jhip.so (built in-tree by deeplearning4j_amd/csrc/Makefile)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise NativeOpsError("%s is missing: build it with `make -C deeplearning4j_amd/csrc` "
                                 "(or __graft_entry__.build()); there is no CPU fallback" % LIB_PATH)
        L = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in _SIGS.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def check(what=""):
    """Poll the error slot the way the Java executioner does after every native call."""
    L = load()
    if L.lastErrorCode() != 0:
        msg = L.lastErrorMessage().decode(errors="replace")
        raise NativeOpsError("%s%s" % (what + ": " if what else "", msg))
