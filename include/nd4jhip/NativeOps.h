/*
 * nd4j-hip: C ABI of the MI355X (gfx950) op backend.
 *
 * Every entry point below replaces the function of the same name in the reference's
 * libnd4j/include/legacy/NativeOps.h (cited as "ref :line" on each declaration).  The reference
 * exports these with C++ linkage and lets JavaCPP parse the C++ header; here they are `extern "C"`
 * with opaque handle types so that any FFI (JavaCPP, JNI, ctypes) can bind them.  Two consequences:
 *   - the reference's C++ overload getShapeInfoLength(OpaqueNDArray) gets the distinct name
 *     getOpaqueNDArrayShapeInfoLength, and of the two lc* overload sets (by value :451-457, by pointer
 *     :500-512) the by-value one keeps the names while the by-pointer one carries the suffix "Ptr"
 *     (lcScalarPointerPtr ...); everything else keeps its name, argument order and meaning;
 *   - handles are plain pointers: OpaqueNDArray = array handle created by createOpaqueNDArray,
 *     OpaqueDataBuffer = host+device buffer pair, OpaqueContext = per-op argument bag.
 *
 * Error convention (ref legacy/cpu/NativeOps.cpp:1118-1121): exec* functions return void; a failure
 * stores {code, message} in a process-wide slot which the caller polls with lastErrorCode() /
 * lastErrorMessage().  execCustomOp2 additionally returns a status (0 = OK).  The slot keeps the last
 * failure until lastErrorMessage() is fetched, which resets the code to 0 (ref
 * execution/impl/ErrorReference.cpp:28-34); successful calls do not touch it.
 *
 * Device model: this library has no CPU execution path.  All compute entry points run HIP kernels on
 * the current device and fail with an error if no device is present.  Arrays carry a host ("primary")
 * and a device ("special") buffer; exec* synchronises host->device lazily by the buffers' read/write
 * stamps (ref array/cuda/DataBuffer.cu:597-606) and marks outputs as written on the device.
 * Legacy exec* calls are asynchronous on the execution stream; execCustomOp2 synchronises before it
 * returns (ref legacy/cuda/NativeOps.cu:118).
 */
#ifndef ND4JHIP_NATIVEOPS_H
#define ND4JHIP_NATIVEOPS_H

#include <stdbool.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ND4JHIP_EXPORT __attribute__((visibility("default")))

typedef long long Nd4jLong;  /* sd::LongType */
typedef void* Nd4jPointer;   /* sd::Pointer */
typedef int Nd4jStatus;      /* sd::Status: 0 = OK, non-zero = failure (ref system/common.h:184-187) */

typedef struct Nd4jHipDataBuffer OpaqueDataBuffer;            /* ref :57  sd::InteropDataBuffer */
typedef struct Nd4jHipNDArray* OpaqueNDArray;                 /* ref :61  sd::NDArray* */
typedef OpaqueNDArray* OpaqueNDArrayArr;                      /* ref :62 */
typedef struct Nd4jHipContext OpaqueContext;                  /* ref :60  sd::graph::Context */
typedef struct Nd4jHipShapeList OpaqueShapeList;              /* ref :59 */
typedef struct Nd4jHipTadPack OpaqueTadPack;                  /* ref :68 */
typedef struct Nd4jHipConstantShapeBuffer* OpaqueConstantShapeBuffer; /* ref :71 */
typedef struct Nd4jHipLaunchContext* OpaqueLaunchContext;     /* ref :63 */

/* dtype codes (ref array/DataType.h:26-50) */
enum Nd4jDataType {
  ND4J_BOOL = 1, ND4J_HALF = 3, ND4J_FLOAT32 = 5, ND4J_DOUBLE = 6, ND4J_INT8 = 7, ND4J_INT16 = 8, ND4J_INT32 = 9,
  ND4J_INT64 = 10, ND4J_UINT8 = 11, ND4J_UINT16 = 12, ND4J_UINT32 = 13, ND4J_UINT64 = 14, ND4J_BFLOAT16 = 17
};

/* ---- library / device -------------------------------------------------------------------------- */
ND4JHIP_EXPORT void initializeDevicesAndFunctions(void);                               /* ref :225 */
ND4JHIP_EXPORT void initializeShapeCache(void);                                        /* ref :238 */
ND4JHIP_EXPORT void initializeTadCache(void);                                          /* ref :252 */
ND4JHIP_EXPORT int getAvailableDevices(void);                                          /* ref :273 */
ND4JHIP_EXPORT int setDevice(int deviceId);                                            /* ref :262 */
ND4JHIP_EXPORT int getDevice(void);                                                    /* ref :318 */
ND4JHIP_EXPORT const char* getDeviceName(int device);                                  /* ref :164 */
ND4JHIP_EXPORT int getDeviceMajor(int device);                                         /* ref :311 */
ND4JHIP_EXPORT int getDeviceMinor(int device);                                         /* ref :312 */
ND4JHIP_EXPORT Nd4jLong getDeviceFreeMemory(int device);                               /* ref :264 */
ND4JHIP_EXPORT Nd4jLong getDeviceFreeMemoryDefault(void);                              /* ref :263 */
ND4JHIP_EXPORT Nd4jLong getDeviceTotalMemory(int device);                              /* ref :265 */
ND4JHIP_EXPORT void enableDebugMode(bool reallyEnable);                                /* ref :274 */
ND4JHIP_EXPORT void enableVerboseMode(bool reallyEnable);                              /* ref :310 */
ND4JHIP_EXPORT void setOmpNumThreads(int threads);                                     /* ref :278 (host threads are not used; kept as a no-op) */
ND4JHIP_EXPORT int ompGetMaxThreads(void);                                             /* ref :276 */
ND4JHIP_EXPORT void setElementThreshold(int num);                                      /* ref :319 (no-op) */
ND4JHIP_EXPORT void setTADThreshold(int num);                                          /* ref :320 (no-op) */
ND4JHIP_EXPORT int lastErrorCode(void);                                                /* ref :553 */
ND4JHIP_EXPORT const char* lastErrorMessage(void);                                     /* ref :552 */

/* memory, streams, events.  Streams travel as pointer-to-handle (hipStream_t*), events as the handle
 * itself, exactly as the reference's device backend does (ref legacy/cuda/NativeOps.cu:1235-1260). */
ND4JHIP_EXPORT Nd4jPointer mallocHost(Nd4jLong memorySize, int flags);                 /* ref :254 (pinned) */
ND4JHIP_EXPORT Nd4jPointer mallocDevice(Nd4jLong memorySize, int deviceId, int flags); /* ref :255 */
ND4JHIP_EXPORT int freeHost(Nd4jPointer pointer);                                      /* ref :256 */
ND4JHIP_EXPORT int freeDevice(Nd4jPointer pointer, int deviceId);                      /* ref :257 */
ND4JHIP_EXPORT Nd4jPointer createStream(void);                                         /* ref :259 */
ND4JHIP_EXPORT Nd4jPointer createEvent(void);                                          /* ref :260 */
ND4JHIP_EXPORT int registerEvent(Nd4jPointer event, Nd4jPointer stream);               /* ref :261 */
ND4JHIP_EXPORT int destroyEvent(Nd4jPointer event);                                    /* ref :270 */
ND4JHIP_EXPORT int streamSynchronize(Nd4jPointer stream);                              /* ref :271 */
ND4JHIP_EXPORT int eventSynchronize(Nd4jPointer event);                                /* ref :272 */
/* flags: 0 host->host, 1 host->device, 2 device->host, 3 device->device; `reserved` = stream (async) */
ND4JHIP_EXPORT int memcpySync(Nd4jPointer dst, Nd4jPointer src, Nd4jLong size, int flags, Nd4jPointer reserved);  /* ref :266 */
ND4JHIP_EXPORT int memcpyAsync(Nd4jPointer dst, Nd4jPointer src, Nd4jLong size, int flags, Nd4jPointer reserved); /* ref :267 */
ND4JHIP_EXPORT int memsetSync(Nd4jPointer dst, int value, Nd4jLong size, int flags, Nd4jPointer reserved);        /* ref :268 */
ND4JHIP_EXPORT int memsetAsync(Nd4jPointer dst, int value, Nd4jLong size, int flags, Nd4jPointer reserved);       /* ref :269 */

/* launch context (ref :451-457,500-512) */
ND4JHIP_EXPORT OpaqueLaunchContext defaultLaunchContext(void);                         /* ref :500 */
ND4JHIP_EXPORT Nd4jPointer lcScalarPointer(OpaqueLaunchContext lc);                    /* ref :451 */
ND4JHIP_EXPORT Nd4jPointer lcReductionPointer(OpaqueLaunchContext lc);                 /* ref :452 */
ND4JHIP_EXPORT Nd4jPointer lcAllocationPointer(OpaqueLaunchContext lc);                /* ref :453 */
ND4JHIP_EXPORT Nd4jPointer lcExecutionStream(OpaqueLaunchContext lc);                  /* ref :454 */
ND4JHIP_EXPORT Nd4jPointer lcCopyStream(OpaqueLaunchContext lc);                       /* ref :455 */
ND4JHIP_EXPORT Nd4jPointer lcBlasHandle(OpaqueLaunchContext lc);                       /* ref :456 (no vendor BLAS is used: returns NULL) */
ND4JHIP_EXPORT Nd4jPointer lcSolverHandle(OpaqueLaunchContext lc);                     /* ref :457 (no vendor solver is used: returns NULL) */
/* the reference's second overload set takes a pointer to the handle (what defaultLaunchContext's Java wrapper holds) */
ND4JHIP_EXPORT Nd4jPointer lcScalarPointerPtr(OpaqueLaunchContext* lc);                /* ref :502 */
ND4JHIP_EXPORT Nd4jPointer lcReductionPointerPtr(OpaqueLaunchContext* lc);             /* ref :504 */
ND4JHIP_EXPORT Nd4jPointer lcAllocationPointerPtr(OpaqueLaunchContext* lc);            /* ref :506 */
ND4JHIP_EXPORT Nd4jPointer lcExecutionStreamPtr(OpaqueLaunchContext* lc);              /* ref :508 */
ND4JHIP_EXPORT Nd4jPointer lcCopyStreamPtr(OpaqueLaunchContext* lc);                   /* ref :510 */
ND4JHIP_EXPORT Nd4jPointer lcBlasHandlePtr(OpaqueLaunchContext* lc);                   /* ref :512 */

/* what a device backend asks at start-up (AtomicAllocator.java:140, CudaAffinityManager.java:353,
 * CudaExecutioner's static initialiser) */
ND4JHIP_EXPORT void checkP2P(void);                                                    /* ref :222 */
ND4JHIP_EXPORT void enableP2P(bool enable);                                            /* ref :223 */
ND4JHIP_EXPORT bool isP2PAvailable(void);                                              /* ref :224 (one device counts as available, ref legacy/cuda/NativeOps.cu:1046-1049) */
ND4JHIP_EXPORT void initializeFunctions(Nd4jPointer* functions);                       /* ref :226 (host BLAS pointers; unused here) */
ND4JHIP_EXPORT bool isBlasVersionMatches(int major, int minor, int build);             /* ref :398 (no vendor BLAS to mismatch: true) */
ND4JHIP_EXPORT int binaryLevel(void);                                                  /* ref :460 */
ND4JHIP_EXPORT int optimalLevel(void);                                                 /* ref :461 */
ND4JHIP_EXPORT bool isMinimalRequirementsMet(void);                                    /* ref :462 */
ND4JHIP_EXPORT bool isOptimalRequirementsMet(void);                                    /* ref :463 */
ND4JHIP_EXPORT bool isExperimentalEnabled(void);                                       /* ref :316 */
ND4JHIP_EXPORT void setOmpMinThreads(int threads);                                     /* ref :317 (no-op) */
ND4JHIP_EXPORT void setGridLimit(int gridSize);                                        /* ref :275 (no-op: grids follow the problem) */
ND4JHIP_EXPORT Nd4jPointer getConstantSpace(void);                                     /* ref :315 (no constant-memory staging area: NULL) */
/* entry points of the reference that lie outside this backend's path: exported so that a binding resolves them; each
 * sets the error slot to "... is not implemented in nd4j-hip" and does nothing else */
ND4JHIP_EXPORT void execRandom(Nd4jPointer* extraPointers, int opNum, Nd4jPointer stateHost, OpaqueNDArray z, void* extraArguments);                  /* ref :166 */
ND4JHIP_EXPORT void execRandom2(Nd4jPointer* extraPointers, int opNum, Nd4jPointer stateHost, OpaqueNDArray x, OpaqueNDArray z, void* extraArguments); /* ref :168 */
ND4JHIP_EXPORT void execRandom3(Nd4jPointer* extraPointers, int opNum, Nd4jPointer stateHost, OpaqueNDArray x, OpaqueNDArray y, OpaqueNDArray z, void* extraArguments); /* ref :170 */
ND4JHIP_EXPORT void sort(Nd4jPointer* extraPointers, OpaqueNDArray x, bool descending);                                                               /* ref :343 */
ND4JHIP_EXPORT void sortTad(Nd4jPointer* extraPointers, OpaqueNDArray x, Nd4jLong* dimension, Nd4jLong dimensionLength, Nd4jLong* tadShapeInfo, Nd4jLong* tadOffsets, bool descending); /* ref :344 */
ND4JHIP_EXPORT void shuffle(Nd4jPointer* extras, OpaqueNDArrayArr x, OpaqueNDArrayArr z, int N, OpaqueNDArray dimension, OpaqueNDArray shuffleMap);   /* ref :84 */
ND4JHIP_EXPORT void pullRows(Nd4jPointer* extraPointers, OpaqueNDArray x, OpaqueNDArray z, Nd4jLong n, OpaqueNDArray indexes, Nd4jLong dimension);    /* ref :95 */
ND4JHIP_EXPORT void convertTypes(Nd4jPointer* extras, int srcType, Nd4jPointer dX, Nd4jLong N, int dstType, Nd4jPointer dZ);                         /* ref :390 */

/* ---- data buffers (ref :466-488) ------------------------------------------------------------------- */
ND4JHIP_EXPORT OpaqueDataBuffer* dbAllocateDataBuffer(Nd4jLong elements, int dataType, bool allocateBoth);        /* ref :487 */
ND4JHIP_EXPORT OpaqueDataBuffer* allocateDataBuffer(Nd4jLong elements, int dataType, bool allocateBoth);          /* ref :497 */
ND4JHIP_EXPORT OpaqueDataBuffer* dbCreateExternalDataBuffer(Nd4jLong elements, int dataType, Nd4jPointer primary, Nd4jPointer special); /* ref :488 */
ND4JHIP_EXPORT OpaqueDataBuffer* dbCreateView(OpaqueDataBuffer* dataBuffer, Nd4jLong length);                     /* ref :486 */
ND4JHIP_EXPORT Nd4jPointer dbPrimaryBuffer(OpaqueDataBuffer* dataBuffer);              /* ref :466 */
ND4JHIP_EXPORT Nd4jPointer dbSpecialBuffer(OpaqueDataBuffer* dataBuffer);              /* ref :467 */
ND4JHIP_EXPORT Nd4jLong dbBufferLength(OpaqueDataBuffer* dataBuffer);                  /* ref :181 */
ND4JHIP_EXPORT void dbSetPrimaryBuffer(OpaqueDataBuffer* dataBuffer, Nd4jPointer primaryBuffer, Nd4jLong numBytes); /* ref :469 */
ND4JHIP_EXPORT void dbSetSpecialBuffer(OpaqueDataBuffer* dataBuffer, Nd4jPointer specialBuffer, Nd4jLong numBytes); /* ref :470 */
ND4JHIP_EXPORT void dbAllocatePrimaryBuffer(OpaqueDataBuffer* dataBuffer);             /* ref :471 */
ND4JHIP_EXPORT void dbAllocateSpecialBuffer(OpaqueDataBuffer* dataBuffer);             /* ref :472 */
ND4JHIP_EXPORT void dbExpandBuffer(OpaqueDataBuffer* dataBuffer, Nd4jLong elements);   /* ref :473 */
ND4JHIP_EXPORT void dbExpand(OpaqueDataBuffer* dataBuffer, Nd4jLong elements);         /* ref :481 */
ND4JHIP_EXPORT int dbUseCount(OpaqueDataBuffer* dataBuffer);                           /* ref :474 */
ND4JHIP_EXPORT void dbSyncToSpecial(OpaqueDataBuffer* dataBuffer);                     /* ref :475 */
ND4JHIP_EXPORT void dbSyncToPrimary(OpaqueDataBuffer* dataBuffer);                     /* ref :476 */
ND4JHIP_EXPORT void dbTickHostRead(OpaqueDataBuffer* dataBuffer);                      /* ref :477 */
ND4JHIP_EXPORT void dbTickHostWrite(OpaqueDataBuffer* dataBuffer);                     /* ref :478 */
ND4JHIP_EXPORT void dbTickDeviceRead(OpaqueDataBuffer* dataBuffer);                    /* ref :479 */
ND4JHIP_EXPORT void dbTickDeviceWrite(OpaqueDataBuffer* dataBuffer);                   /* ref :480 */
ND4JHIP_EXPORT void dbClose(OpaqueDataBuffer* dataBuffer);                             /* ref :482 */
ND4JHIP_EXPORT int dbDeviceId(OpaqueDataBuffer* dataBuffer);                           /* ref :483 */
ND4JHIP_EXPORT void dbSetDeviceId(OpaqueDataBuffer* dataBuffer, int deviceId);         /* ref :484 */
ND4JHIP_EXPORT int dbLocality(OpaqueDataBuffer* dataBuffer);                           /* ref :485: -1 host current, 1 device current, 0 both */
ND4JHIP_EXPORT void deleteDataBuffer(OpaqueDataBuffer* dataBuffer);                    /* ref :468 */

/* ---- shape descriptors (ref :490-495, :395-404) ------------------------------------------------------ */
ND4JHIP_EXPORT OpaqueConstantShapeBuffer shapeBuffer(int rank, Nd4jLong* shape, Nd4jLong* strides, int dtype, char order, Nd4jLong ews, bool empty); /* ref :491 */
ND4JHIP_EXPORT OpaqueConstantShapeBuffer shapeBufferEx(int rank, Nd4jLong* shape, Nd4jLong* strides, int dtype, char order, Nd4jLong ews, Nd4jLong extras); /* ref :493 */
ND4JHIP_EXPORT OpaqueConstantShapeBuffer cacheAndStoreShapeBuffer(Nd4jLong* shapeInfo);                           /* ref :490 */
ND4JHIP_EXPORT Nd4jPointer getConstantShapeBufferPrimary(OpaqueConstantShapeBuffer dbf);                          /* ref :403 */
ND4JHIP_EXPORT Nd4jPointer getConstantShapeBufferSpecial(OpaqueConstantShapeBuffer dbf);                          /* ref :404 */
ND4JHIP_EXPORT void deleteConstantShapeBuffer(OpaqueConstantShapeBuffer* ptr);                                    /* ref :395 (cache-owned: no-op) */

/* ---- array handles (ref :111-125, :336-342) ------------------------------------------------------------ */
ND4JHIP_EXPORT OpaqueNDArray createOpaqueNDArray(OpaqueDataBuffer* shapeInfo, OpaqueDataBuffer* buffer, OpaqueDataBuffer* specialBuffer, Nd4jLong offset); /* ref :122 */
ND4JHIP_EXPORT void deleteNDArray(OpaqueNDArray array);                                /* ref :111 */
ND4JHIP_EXPORT Nd4jLong getOpaqueNDArrayOffset(OpaqueNDArray array);                   /* ref :113 */
ND4JHIP_EXPORT const Nd4jLong* getOpaqueNDArrayShapeInfo(OpaqueNDArray array);         /* ref :116 */
ND4JHIP_EXPORT void* getOpaqueNDArrayBuffer(OpaqueNDArray array);                      /* ref :118 */
ND4JHIP_EXPORT void* getOpaqueNDArraySpecialBuffer(OpaqueNDArray array);               /* ref :120 */
ND4JHIP_EXPORT Nd4jLong getOpaqueNDArrayLength(OpaqueNDArray array);                   /* ref :342 */
ND4JHIP_EXPORT Nd4jLong getOpaqueNDArrayShapeInfoLength(OpaqueNDArray array);          /* ref :341 getShapeInfoLength(OpaqueNDArray) */

/* ---- TAD packs (ref :142-159, :397) ---------------------------------------------------------------------- */
ND4JHIP_EXPORT OpaqueTadPack* tadOnlyShapeInfo(OpaqueDataBuffer* hXShapeInfo, Nd4jLong* dimension, Nd4jLong dimensionLength); /* ref :159 */
ND4JHIP_EXPORT const Nd4jLong* getPrimaryShapeInfo(OpaqueTadPack* pack);               /* ref :142 */
ND4JHIP_EXPORT const Nd4jLong* getPrimaryOffsets(OpaqueTadPack* pack);                 /* ref :143 */
ND4JHIP_EXPORT const Nd4jLong* getSpecialShapeInfo(OpaqueTadPack* pack);               /* ref :144 */
ND4JHIP_EXPORT const Nd4jLong* getSpecialOffsets(OpaqueTadPack* pack);                 /* ref :145 */
ND4JHIP_EXPORT Nd4jLong getNumberOfTads(OpaqueTadPack* pack);                          /* ref :146 */
ND4JHIP_EXPORT int getShapeInfoLength(OpaqueTadPack* pack);                            /* ref :147 */
ND4JHIP_EXPORT void deleteTadPack(OpaqueTadPack* ptr);                                 /* ref :397 (cache-owned: no-op) */

/* ---- legacy loops ------------------------------------------------------------------------------------------ */
ND4JHIP_EXPORT void execPairwiseTransform(Nd4jPointer* extraPointers, int opNum, OpaqueNDArray x, OpaqueNDArray y, OpaqueNDArray z, void* extraParams); /* ref :195 */
ND4JHIP_EXPORT void execTransformStrict(Nd4jPointer* extraPointers, int opNum, OpaqueNDArray x, void* extraParams, OpaqueNDArray z); /* ref :220 */
ND4JHIP_EXPORT void execTransformFloat(Nd4jPointer* extraPointers, int opNum, OpaqueNDArray x, void* extraParams, OpaqueNDArray z);  /* ref :221 */
ND4JHIP_EXPORT void execTransformSame(Nd4jPointer* extraPointers, int opNum, OpaqueNDArray x, void* extraParams, OpaqueNDArray z);   /* ref :217 */
ND4JHIP_EXPORT void execTransformAny(Nd4jPointer* extraPointers, int opNum, OpaqueNDArray x, void* extraParams, OpaqueNDArray z);    /* ref :219 */
ND4JHIP_EXPORT void execReduceFloat(Nd4jPointer* extraPointers, int opNum, OpaqueNDArray x, void* extraParams, OpaqueNDArray z);     /* ref :207 */
ND4JHIP_EXPORT void execReduceFloat2(Nd4jPointer* extraPointers, int opNum, OpaqueNDArray x, void* extraParams, OpaqueNDArray z, OpaqueNDArray dimension); /* ref :215 */
ND4JHIP_EXPORT void execReduceSame(Nd4jPointer* extraPointers, int opNum, OpaqueNDArray x, void* extraParams, OpaqueNDArray z);      /* ref :321 */
ND4JHIP_EXPORT void execReduceSame2(Nd4jPointer* extraPointers, int opNum, OpaqueNDArray x, void* extraParams, OpaqueNDArray z, OpaqueNDArray dimension);  /* ref :323 */
ND4JHIP_EXPORT void execIndexReduce(Nd4jPointer* extraPointers, int opNum, OpaqueNDArray x, void* extraParams, OpaqueNDArray z, OpaqueNDArray dimension);  /* ref :214 */
ND4JHIP_EXPORT void execIndexReduceScalar(Nd4jPointer* extraPointers, int opNum, OpaqueNDArray x, void* extraParams, OpaqueNDArray z); /* ref :216 */
ND4JHIP_EXPORT void execScalar(Nd4jPointer* extraPointers, int opNum, OpaqueNDArray x, OpaqueNDArray z, OpaqueNDArray scalar, void* extraParams); /* ref :204 */
ND4JHIP_EXPORT void execTransformBool(Nd4jPointer* extraPointers, int opNum, OpaqueNDArray x, void* extraParams, OpaqueNDArray z);   /* ref :218 */
ND4JHIP_EXPORT void execSummaryStatsScalar(Nd4jPointer* extraPointers, int opNum, OpaqueNDArray x, void* extraParams, OpaqueNDArray z, bool biasCorrected); /* ref :197 */
ND4JHIP_EXPORT void execSummaryStatsTad(Nd4jPointer* extraPointers, int opNum, OpaqueNDArray x, void* extraParams, OpaqueNDArray z, OpaqueNDArray dimension, bool biasCorrected); /* ref :198-199 */
ND4JHIP_EXPORT void execReduce3(Nd4jPointer* extraPointers, int opNum, OpaqueNDArray x, void* extraParams, OpaqueNDArray y, OpaqueNDArray z);        /* ref :326 */
ND4JHIP_EXPORT void execReduce3Scalar(Nd4jPointer* extraPointers, int opNum, OpaqueNDArray x, void* extraParams, OpaqueNDArray y, OpaqueNDArray z);  /* ref :327 */
ND4JHIP_EXPORT void execReduce3Tad(Nd4jPointer* extraPointers, int opNum, OpaqueNDArray x, void* extraParams, OpaqueNDArray y, OpaqueNDArray z, OpaqueNDArray dimension); /* ref :328 */
/* every sub-array of x along `dimension` against every sub-array of y along it: z[i][j], shape [sub-arrays of x, sub-arrays of y] */
ND4JHIP_EXPORT void execReduce3All(Nd4jPointer* extraPointers, int opNum, OpaqueNDArray x, OpaqueNDArray y, OpaqueNDArray z, OpaqueNDArray dimension, void* extraParams); /* ref :208 */
ND4JHIP_EXPORT void execReduceLong(Nd4jPointer* extraPointers, int opNum, OpaqueNDArray x, void* extraParams, OpaqueNDArray z, OpaqueNDArray dimension);  /* ref :211 */
ND4JHIP_EXPORT void execReduceLong2(Nd4jPointer* extraPointers, int opNum, OpaqueNDArray x, void* extraParams, OpaqueNDArray z, OpaqueNDArray dimension); /* ref :349-351 */
ND4JHIP_EXPORT void execReduceBool(Nd4jPointer* extraPointers, int opNum, OpaqueNDArray x, void* extraParams, OpaqueNDArray z, OpaqueNDArray dimension);  /* ref :213 */
ND4JHIP_EXPORT void execReduceBool2(Nd4jPointer* extraPointers, int opNum, OpaqueNDArray x, void* extraParams, OpaqueNDArray z, OpaqueNDArray dimension); /* ref :212 */
ND4JHIP_EXPORT void execBroadcast(Nd4jPointer* extraPointers, int opNum, OpaqueNDArray x, OpaqueNDArray y, OpaqueNDArray z, void* extraParams, OpaqueNDArray dimension); /* ref :206 */
/* The bool tables (loops/legacy_ops.h:30-32, 74-76, 117-119): x and y (or the scalar) of one type, z BOOL.  EqualTo, GreaterThan,
 * LessThan, Epsilon, GreaterThanOrEqual, NotEqualTo, And, Or, Xor, Not, LessThanOrEqual; 5 (MatchCondition) is refused.
 * Epsilon / And / Or / Xor read one extra parameter when extraParams is not null (held in x's type, fetched with a blocking copy). */
ND4JHIP_EXPORT void execPairwiseTransformBool(Nd4jPointer* extraPointers, int opNum, OpaqueNDArray x, OpaqueNDArray y, void* extraParams, OpaqueNDArray z); /* ref :196 */
ND4JHIP_EXPORT void execBroadcastBool(Nd4jPointer* extraPointers, int opNum, OpaqueNDArray x, OpaqueNDArray y, OpaqueNDArray z, void* extraParams, OpaqueNDArray dimension); /* ref :200 */
ND4JHIP_EXPORT void execScalarBool(Nd4jPointer* extraPointers, int opNum, OpaqueNDArray x, OpaqueNDArray z, OpaqueNDArray scalar, void* extraParams); /* ref :201 */
/* One scalar per sub-array of x along `dimension` (the scalars numbered in c order over x's other dims). */
ND4JHIP_EXPORT void execScalarBoolTad(Nd4jPointer* extraPointers, int opNum, OpaqueNDArray x, OpaqueNDArray z, OpaqueNDArray scalars, void* extraParams, OpaqueNDArray dimension); /* ref :203 */
ND4JHIP_EXPORT void execScalarTad(Nd4jPointer* extraPointers, int opNum, OpaqueNDArray x, OpaqueNDArray z, OpaqueNDArray scalars, void* extraParams, OpaqueNDArray dimension); /* ref :205 */

/* ---- op context + declarable ops ---------------------------------------------------------------------------- */
ND4JHIP_EXPORT const char* getAllCustomOps(void);                                      /* ref :76 */
ND4JHIP_EXPORT OpaqueContext* createGraphContext(int nodeId);                          /* ref :79 */
ND4JHIP_EXPORT void deleteGraphContext(OpaqueContext* ptr);                            /* ref :437 */
ND4JHIP_EXPORT void markGraphContextInplace(OpaqueContext* ptr, bool reallyInplace);   /* ref :416 */
ND4JHIP_EXPORT void setGraphContextInputArray(OpaqueContext* ptr, int index, OpaqueNDArray arr);   /* ref :430 */
ND4JHIP_EXPORT void setGraphContextOutputArray(OpaqueContext* ptr, int index, OpaqueNDArray arr);  /* ref :429 */
ND4JHIP_EXPORT void setGraphContextInputArraysArr(OpaqueContext* ptr, int numArrays, OpaqueNDArrayArr arr);  /* ref :432 */
ND4JHIP_EXPORT void setGraphContextOutputArraysArr(OpaqueContext* ptr, int numArrays, OpaqueNDArrayArr arr); /* ref :431 */
ND4JHIP_EXPORT void setGraphContextTArguments(OpaqueContext* ptr, double* arguments, int numberOfArguments);   /* ref :433 */
ND4JHIP_EXPORT void setGraphContextIArguments(OpaqueContext* ptr, Nd4jLong* arguments, int numberOfArguments); /* ref :434 */
ND4JHIP_EXPORT void setGraphContextBArguments(OpaqueContext* ptr, bool* arguments, int numberOfArguments);     /* ref :435 */
/* The caller's stream (pointer to it, as lcExecutionStream returns) and scratch for this op (ref CudaOpContext.java:291).  Work queued
 * on that stream is ordered before the op and the op before what the caller queues next; kernels run on the library's own
 * execution stream and use its own scratch. */
ND4JHIP_EXPORT void setGraphContextCudaContext(OpaqueContext* ptr, void* stream, void* reductionPointer, void* allocationPointer);  /* ref :80 */
ND4JHIP_EXPORT void setGraphContextDArguments(OpaqueContext* ptr, int* arguments, int numberOfArguments);      /* ref :436 */
ND4JHIP_EXPORT void ctxAllowHelpers(OpaqueContext* ptr, bool reallyAllow);             /* ref :464 */
ND4JHIP_EXPORT void ctxShapeFunctionOverride(OpaqueContext* ptr, bool reallyOverride); /* ref :458 */
ND4JHIP_EXPORT void ctxSetExecutionMode(OpaqueContext* ptr, int execMode);             /* ref :465 */
ND4JHIP_EXPORT void ctxPurge(OpaqueContext* ptr);                                      /* ref :459 */
ND4JHIP_EXPORT OpaqueNDArray getInputArrayNative(OpaqueContext* ptr, int idx);         /* ref :418 */
ND4JHIP_EXPORT OpaqueNDArray getOutputArrayNative(OpaqueContext* ptr, int idx);        /* ref :417 */
ND4JHIP_EXPORT Nd4jLong numInputsNative(OpaqueContext* ptr);                           /* ref :425 */
ND4JHIP_EXPORT Nd4jLong numOutputsNative(OpaqueContext* ptr);                          /* ref :424 */
ND4JHIP_EXPORT Nd4jLong numTArgumentsNative(OpaqueContext* ptr);                       /* ref :427 */
ND4JHIP_EXPORT Nd4jLong numIArgumentsNative(OpaqueContext* ptr);                       /* ref :428 */
ND4JHIP_EXPORT Nd4jLong numBNative(OpaqueContext* ptr);                                /* ref :423 */
ND4JHIP_EXPORT Nd4jLong numDNative(OpaqueContext* ptr);                                /* ref :422 */
ND4JHIP_EXPORT double tArgumentNative(OpaqueContext* ptr, int idx);                    /* ref :426 */
ND4JHIP_EXPORT Nd4jLong iArgumentAtNative(OpaqueContext* ptr, int idx);                /* ref :421 */
ND4JHIP_EXPORT bool bArgAtNative(OpaqueContext* ptr, int idx);                         /* ref :420 */
ND4JHIP_EXPORT Nd4jLong dataTypeNativeAt(OpaqueContext* ptr, int idx);                 /* ref :419 */
ND4JHIP_EXPORT Nd4jStatus execCustomOp2(Nd4jPointer* extraPointers, Nd4jLong hash, OpaqueContext* opContext);  /* ref :370 */
ND4JHIP_EXPORT OpaqueShapeList* calculateOutputShapes2(Nd4jPointer* extraPointers, Nd4jLong hash, OpaqueContext* context); /* ref :176 */
ND4JHIP_EXPORT Nd4jLong getShapeListSize(OpaqueShapeList* list);                       /* ref :177 */
ND4JHIP_EXPORT const Nd4jLong* getShape(OpaqueShapeList* list, Nd4jLong i);            /* ref :174 */
ND4JHIP_EXPORT void deleteShapeList(Nd4jPointer shapeList);                            /* ref :386 */

/* ---- additions without a counterpart in the reference ------------------------------------------------------- */
/* 64-bit hash of an op name, the key execCustomOp2 takes (ref helpers/impl/helper_hash.cpp:33-70 computes it
 * inside the library only; callers normally parse it out of getAllCustomOps()). */
ND4JHIP_EXPORT Nd4jLong nd4jhipOpHash(const char* opName);
/* Events that record time, for benchmarks: createEvent() above disables timing like the reference does. */
ND4JHIP_EXPORT Nd4jPointer nd4jhipCreateTimingEvent(void);
ND4JHIP_EXPORT float nd4jhipEventElapsedMs(Nd4jPointer startEvent, Nd4jPointer stopEvent);
/* 1: execCustomOp2 synchronises the stream before returning (default, reference behaviour); 0: the caller
 * synchronises itself (streamSynchronize / dbSyncToPrimary) -- used by tight decode loops. */
ND4JHIP_EXPORT void nd4jhipSetSyncAfterCustomOp(int enable);
/* Stream capture for launch-bound op sequences (a decode step is ~150 kernels of a few microseconds each): every op
 * call between Begin and End is recorded on the execution stream instead of run; End returns a handle (null + error slot
 * when an op waited on the stream, copied synchronously or allocated, which invalidates a capture); Launch replays the
 * recorded kernels with the arguments they were recorded with.  Build arrays, views and OpContexts before Begin.
 * Handle lifetime: every recorded call copies its array views (shape, strides, offset; the DataBuffers are shared) the
 * moment it is recorded, so array handles and OpContexts may be deleted right after the op call that used them, before
 * End; the DataBuffers must outlive the graph.  memcpyAsync (device to device) and memsetAsync on the library's stream
 * (a null `reserved`, or what lcExecutionStream returned) between Begin and End are recorded too and replay in both
 * replay modes; a copy that touches host memory there is an error.
 * Launch keeps the buffers' host/device stamps as the recorded op calls would: a buffer the graph reads whose host copy
 * is newer is uploaded first, and every buffer the graph writes counts as device-written afterwards, so dbSyncToPrimary
 * after a replay returns that replay's values.  A capture is process-wide: ops other threads issue between Begin and End
 * are recorded too. */
ND4JHIP_EXPORT int nd4jhipGraphBeginCapture(void);
ND4JHIP_EXPORT Nd4jPointer nd4jhipGraphEndCapture(void);
ND4JHIP_EXPORT int nd4jhipGraphLaunch(Nd4jPointer graph);
ND4JHIP_EXPORT void nd4jhipGraphDestroy(Nd4jPointer graph);
/* When every op call of a capture is one the library keeps a record of (execCustomOp2, execPairwiseTransform,
 * execTransformStrict, execTransformAny), End replays the recorded calls through a merging pass before it builds the graph:
 * a pairwise Add and the layer_norm of its result become one kernel, and so do xw_plus_b and the GELU transform / the
 * column-slice assigns that follow it.  Every merged kernel writes what the separate ops would have written, bit for
 * bit, into the same arrays.  This returns how many op calls were absorbed that way (0: the graph holds the calls as
 * made).  ND4JHIP_GRAPH_FUSION=0 in the environment switches the pass off. */
ND4JHIP_EXPORT int nd4jhipGraphFusedOps(Nd4jPointer graph);
/* The count above is taken when the merged plan is laid out.  A merged step still asks its kernel at run time whether it
 * takes the operands it meets (alignment, strides) and runs the ops apart when it does not.  This returns how many op
 * calls did run inside a neighbour's kernel the last time the plan was executed: while End re-recorded it, or on the
 * latest kernel-by-kernel replay.  Equal to nd4jhipGraphFusedOps when every merged kernel ran. */
ND4JHIP_EXPORT int nd4jhipGraphFusedApplied(Nd4jPointer graph);
/* How nd4jhipGraphLaunch replays a recording (no counterpart in the reference, like the capture calls themselves).
 * 0: the instantiated HIP graph, one launch.  1: the recorded, merged sequence launched kernel by kernel on the execution
 * stream by the library itself -- the same kernels with the same arguments, without the caller's per-op calls; a kernel
 * tracer then sees the merged step as ordinary dispatches, and on hosts where a graph launch costs more per node than a
 * plain launch it is also the faster of the two.  A recording made while some call went unrecorded has no such sequence
 * and is always launched as a graph.  The recording keeps its own views of the arrays (the buffers are shared), so the
 * caller's array handles may go away in either mode; the buffers may not.  The setting is process-wide and read at
 * every launch; it starts as 0, or 1 when ND4JHIP_GRAPH_REPLAY=kernels is in the environment.
 * One exception to mode 0: when a rocprofiler tool library is attached to the process (ROCP_TOOL_LIBRARIES or LD_PRELOAD
 * names it, or it is among the loaded objects -- nd4jhipProfilerAttached() returns 1), nd4jhipGraphLaunch replays the
 * recorded plan as in mode 1 whatever the setting, and fails for a recording that has no plan: a graph launch under the
 * kernel tracer once aborted the queue, the cause was never established, and the library keeps callers off that path. */
ND4JHIP_EXPORT void nd4jhipSetGraphReplayMode(int mode);
ND4JHIP_EXPORT int nd4jhipGetGraphReplayMode(void);
ND4JHIP_EXPORT int nd4jhipProfilerAttached(void);
/* Host-side audit of a recording: walks the graph's kernel nodes and checks each one's block size, dynamic LDS request and
 * grid against what the runtime reports for the function and the device.  Launches nothing.  Returns the number of nodes
 * that break a limit (described in the error slot), 0 for a clean graph, -1 when the graph cannot be walked. */
ND4JHIP_EXPORT int nd4jhipGraphAudit(Nd4jPointer graph);
ND4JHIP_EXPORT const char* nd4jhipBuildInfo(void);
/* Name ("family<type,tile,flags>") of the kernel the calling thread's most recent matmul / xw_plus_b launched; lets a
 * test assert that its shape reached the instantiation it means to check. */
ND4JHIP_EXPORT const char* nd4jhipLastGemmKernel(void);
/* The order in which the fused attention kernels take the query tiles of a causal launch when all of its blocks are on
 * the chip at once: items[blockId] = queryTileFromTheEnd * batchEntries + batchEntry, laid out on the host so that the
 * block ids that share a CU (id mod 256) carry about the same number of key tiles and, with a multiple of 8 batch
 * entries, a batch entry stays on one XCD (id mod 8).  Fills `items` (room for batchEntries * queryTiles values) and
 * returns their number, or 0 when such a launch takes the plain heavy-first order instead (more blocks than
 * 256 * residentBlocksPerCu or than the table holds, or at most one block per CU).  Pure host arithmetic: launches
 * nothing and needs no device; lets a test check the layout the kernels are handed. */
ND4JHIP_EXPORT int nd4jhipAttentionBlockOrder(int batchEntries, int queryTiles, int keyTilesPerQueryTile, int residentBlocksPerCu,
                                              unsigned short* items);

/* execReduceSame's full reduction for callers that cannot allocate.  No counterpart in the reference: it is for code
 * under HIP graph capture, tight serving loops and harnesses that forbid hipMalloc.  z[0] = reduce(x[0 .. length)) for
 * a dense device array x of `dataType` (FLOAT, DOUBLE, HALF, BFLOAT16) and the opNums of execReduceSame (0 Sum, 1 Max,
 * 2 Min, 3 Prod, 4 ASum, 5 AMax, 6 AMin); same kernels as execReduceSame, hence the same bits.  dX / dZ are device
 * pointers; stream is a pointer to the caller's stream as lcExecutionStream returns it, or null for the library's own.
 * The cross-block partials go to a fixed 64 KiB device array inside the library (one copy per device, held until the
 * process ends) instead of allocated scratch, and the call allocates nothing, on the error paths either.  Limits:
 * 1 <= length <= 2^31 - 1 (larger: error); initializeDevicesAndFunctions must have run (it allocates; this call
 * refuses to); calls that overlap on one device share the array and race.  Under a caller's own stream capture pass
 * that stream; between nd4jhipGraphBeginCapture and End a null stream is the capturing stream, and the launches become
 * nodes of that recording (which then replays as a graph only: the call leaves no step in the kernel-by-kernel plan).
 * Returns 0, or 1 with the error slot set. */
ND4JHIP_EXPORT int nd4jhipReduceSameScalarNoAlloc(Nd4jPointer stream, int opNum, int dataType, const void* dX, Nd4jLong length, void* dZ);

#ifdef __cplusplus
}
#endif
#endif /* ND4JHIP_NATIVEOPS_H */
