// The C-ABI facade: handle types, buffers, descriptors, device utilities and the legacy exec* loops.
// Every function catches exceptions and records them in the error slot, the way the reference's
// facade does (libnd4j/include/legacy/cpu/NativeOps.cpp:1118-1121).
#include "../../include/nd4jhip/NativeOps.h"

#include <cstring>
#include <link.h>

#include "custom_ops.h"
#include "kernels.h"
#include "plan.h"
#include "runtime.h"

using namespace nd4jhip;

struct Nd4jHipDataBuffer : public InteropDataBuffer {};
struct Nd4jHipNDArray : public NDArray {};
struct Nd4jHipContext : public Context {};
struct Nd4jHipShapeList : public ShapeList {};
struct Nd4jHipTadPack : public TadPack {};
struct Nd4jHipConstantShapeBuffer : public ConstantShapeBuffer {};
struct Nd4jHipLaunchContext : public LaunchContext {};

#define GUARD_BEGIN try {
#define GUARD_END(ret)                         \
  }                                            \
  catch (std::exception & e) {                 \
    errorRef().set(1, e.what());               \
    return ret;                                \
  }                                            \
  catch (...) {                                \
    errorRef().set(1, "unknown native error"); \
    return ret;                                \
  }
#define GUARD_END_VOID GUARD_END()

// Every compute entry point runs under one process-wide lock: the library has one execution stream and one pair of
// scratch buffers, and an op may be several launches that share scratch (split-K partial tiles and their finishing
// kernel, cross-block reduction partials), so two caller threads must not interleave inside an op.
static std::recursive_mutex& opMutex() {
  static std::recursive_mutex m;
  return m;
}
// The caller's stream, when it hands one in (extraPointers[1] of the legacy loops, setGraphContextCudaContext for
// declarable ops; a device backend passes what lcExecutionStream returned, ref CudaExecutioner.java:641-649): work the
// caller queued there is ordered before the op, and the op before whatever the caller queues next.  A null slot or the
// library's own stream needs nothing.
static int* g_captureOpCalls = nullptr;   // while a capture is open: how many op entry points were called
struct OpScope {
  std::lock_guard<std::recursive_mutex> lock;
  hipStream_t caller = nullptr;
  explicit OpScope(void* streamPtr, bool isOp = true) : lock(opMutex()) {
    if (isOp && g_captureOpCalls && captureActive()) ++*g_captureOpCalls;
    if (streamPtr == nullptr || captureActive()) return;
    hipStream_t cs = *reinterpret_cast<hipStream_t*>(streamPtr);
    LaunchContext* lc = LaunchContext::defaultContext();
    if (cs == nullptr || cs == lc->execStream) return;
    caller = cs;
    HIP_CHECK(hipEventRecord(lc->bridgeIn, caller));
    HIP_CHECK(hipStreamWaitEvent(lc->execStream, lc->bridgeIn, 0));
  }
  ~OpScope() {
    if (!caller) return;
    LaunchContext* lc = LaunchContext::defaultContext();
    if (hipEventRecord(lc->bridgeOut, lc->execStream) == hipSuccess) (void)hipStreamWaitEvent(caller, lc->bridgeOut, 0);
  }
};
static void* callerStream(Nd4jPointer* extraPointers) { return extraPointers ? extraPointers[1] : nullptr; }
#define OP_BEGIN(streamPtr) try { OpScope _opScope(streamPtr);
#define GRAPH_BEGIN try { OpScope _opScope(nullptr, false);
static void recordOp(RecordedOp&& r);
static void transformStrictImpl(int opNum, NDArray* x, void* extraParams, NDArray* z);
static void pairwiseImpl(int opNum, NDArray* x, NDArray* y, NDArray* z);

static NDArray* arr(OpaqueNDArray a, const char* fn, const char* name) {
  if (a == nullptr) ND4J_THROW(std::string(fn) + ": " + name + " is null");
  return static_cast<NDArray*>(a);
}
static hipStream_t execStream() { return LaunchContext::defaultContext()->execStream; }

extern "C" {

// ---- library / device ------------------------------------------------------------------------------
void initializeDevicesAndFunctions(void) {
  GUARD_BEGIN
  LaunchContext::defaultContext();
  (void)reduceNoAllocScratch();   // address of the fixed partials array on this device, for nd4jhipReduceSameScalarNoAlloc
  GUARD_END_VOID
}
void initializeShapeCache(void) {}
void initializeTadCache(void) {}
int getAvailableDevices(void) {
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess) { (void)hipGetLastError(); return 0; }
  return n;
}
int setDevice(int deviceId) {
  GUARD_BEGIN
  HIP_CHECK(hipSetDevice(deviceId));
  return 1;
  GUARD_END(0)
}
int getDevice(void) {
  int d = 0;
  if (hipGetDevice(&d) != hipSuccess) { (void)hipGetLastError(); return 0; }
  return d;
}
const char* getDeviceName(int device) {
  static thread_local char name[256];
  hipDeviceProp_t p;
  if (hipGetDeviceProperties(&p, device) != hipSuccess) { (void)hipGetLastError(); return "unknown"; }
  snprintf(name, sizeof(name), "%s (%s)", p.name, p.gcnArchName);
  return name;
}
int getDeviceMajor(int device) {
  hipDeviceProp_t p;
  if (hipGetDeviceProperties(&p, device) != hipSuccess) { (void)hipGetLastError(); return 0; }
  return p.major;
}
int getDeviceMinor(int device) {
  hipDeviceProp_t p;
  if (hipGetDeviceProperties(&p, device) != hipSuccess) { (void)hipGetLastError(); return 0; }
  return p.minor;
}
Nd4jLong getDeviceFreeMemory(int device) {
  GUARD_BEGIN
  int cur = 0;
  HIP_CHECK(hipGetDevice(&cur));
  if (device >= 0 && device != cur) HIP_CHECK(hipSetDevice(device));
  size_t f = 0, t = 0;
  HIP_CHECK(hipMemGetInfo(&f, &t));
  if (device >= 0 && device != cur) HIP_CHECK(hipSetDevice(cur));
  return (Nd4jLong)f;
  GUARD_END(0)
}
Nd4jLong getDeviceFreeMemoryDefault(void) { return getDeviceFreeMemory(-1); }
Nd4jLong getDeviceTotalMemory(int device) {
  hipDeviceProp_t p;
  if (hipGetDeviceProperties(&p, device) != hipSuccess) { (void)hipGetLastError(); return 0; }
  return (Nd4jLong)p.totalGlobalMem;
}
void enableDebugMode(bool e) { Environment::get().debug = e; }
void enableVerboseMode(bool e) { Environment::get().verbose = e; }
void setOmpNumThreads(int) {}
int ompGetMaxThreads(void) { return 1; }
void setElementThreshold(int) {}
void setTADThreshold(int) {}
int lastErrorCode(void) {
  std::lock_guard<std::mutex> g(errorRef().lock);
  return errorRef().code;
}
const char* lastErrorMessage(void) {
  // fetching the message consumes the error: the code goes back to 0 (execution/impl/ErrorReference.cpp:28-34)
  static thread_local std::string copy;
  std::lock_guard<std::mutex> g(errorRef().lock);
  copy = errorRef().message;
  errorRef().code = 0;
  return copy.c_str();
}

Nd4jPointer mallocHost(Nd4jLong memorySize, int) {
  GUARD_BEGIN
  void* p = nullptr;
  HIP_CHECK(hipHostMalloc(&p, (size_t)memorySize + 8, hipHostMallocDefault));
  return p;
  GUARD_END(nullptr)
}
Nd4jPointer mallocDevice(Nd4jLong memorySize, int, int) {
  GUARD_BEGIN
  void* p = nullptr;
  HIP_CHECK(hipMalloc(&p, (size_t)memorySize + 8));
  return p;
  GUARD_END(nullptr)
}
int freeHost(Nd4jPointer pointer) {
  GUARD_BEGIN
  HIP_CHECK(hipHostFree(pointer));
  return 1;
  GUARD_END(0)
}
int freeDevice(Nd4jPointer pointer, int) {
  GUARD_BEGIN
  HIP_CHECK(hipFree(pointer));
  return 1;
  GUARD_END(0)
}
Nd4jPointer createStream(void) {
  GUARD_BEGIN
  auto* s = new hipStream_t;
  HIP_CHECK(hipStreamCreateWithFlags(s, hipStreamNonBlocking));
  return s;
  GUARD_END(nullptr)
}
Nd4jPointer createEvent(void) {
  GUARD_BEGIN
  hipEvent_t e;
  HIP_CHECK(hipEventCreateWithFlags(&e, hipEventDisableTiming));
  return (Nd4jPointer)e;
  GUARD_END(nullptr)
}
Nd4jPointer nd4jhipCreateTimingEvent(void) {
  GUARD_BEGIN
  hipEvent_t e;
  HIP_CHECK(hipEventCreate(&e));
  return (Nd4jPointer)e;
  GUARD_END(nullptr)
}
float nd4jhipEventElapsedMs(Nd4jPointer a, Nd4jPointer b) {
  GUARD_BEGIN
  float ms = 0;
  HIP_CHECK(hipEventElapsedTime(&ms, (hipEvent_t)a, (hipEvent_t)b));
  return ms;
  GUARD_END(-1.f)
}
static hipStream_t streamOf(Nd4jPointer p) { return p ? *reinterpret_cast<hipStream_t*>(p) : execStream(); }
int registerEvent(Nd4jPointer event, Nd4jPointer stream) {
  GUARD_BEGIN
  HIP_CHECK(hipEventRecord((hipEvent_t)event, streamOf(stream)));
  return 1;
  GUARD_END(0)
}
int destroyEvent(Nd4jPointer event) {
  GUARD_BEGIN
  HIP_CHECK(hipEventDestroy((hipEvent_t)event));
  return 1;
  GUARD_END(0)
}
int streamSynchronize(Nd4jPointer stream) {
  GUARD_BEGIN
  HIP_CHECK(hipStreamSynchronize(streamOf(stream)));
  return 1;
  GUARD_END(0)
}
int eventSynchronize(Nd4jPointer event) {
  GUARD_BEGIN
  HIP_CHECK(hipEventSynchronize((hipEvent_t)event));
  return 1;
  GUARD_END(0)
}
static hipMemcpyKind kindOf(int flags) {
  switch (flags) {
    case 0: return hipMemcpyHostToHost;
    case 1: return hipMemcpyHostToDevice;
    case 2: return hipMemcpyDeviceToHost;
    case 3: return hipMemcpyDeviceToDevice;
    default: ND4J_THROW("UNDEFINED MEMCPY");
  }
}
int memcpySync(Nd4jPointer dst, Nd4jPointer src, Nd4jLong size, int flags, Nd4jPointer) {
  GUARD_BEGIN
  HIP_CHECK(hipMemcpy(dst, src, (size_t)size, kindOf(flags)));
  return 1;
  GUARD_END(0)
}
// memcpyAsync / memsetAsync on the library's own stream while a capture is open are part of the recording: they run
// under the op lock, count as op calls and leave a RAW record, so that a recording that holds them replays them in
// both replay modes (as a graph node, and as a step of the kernel-by-kernel plan).  Only device-to-device copies can be
// recorded; a copy that touches host memory inside a capture is an error.
static bool rawOpInCapture(hipStream_t st) { return captureActive() && g_captureOpCalls != nullptr && st == execStream(); }
int memcpyAsync(Nd4jPointer dst, Nd4jPointer src, Nd4jLong size, int flags, Nd4jPointer reserved) {
  GRAPH_BEGIN
  const hipStream_t st = streamOf(reserved);
  const hipMemcpyKind kind = kindOf(flags);
  const bool recorded = rawOpInCapture(st);
  if (recorded) ND4J_REQUIRE(kind == hipMemcpyDeviceToDevice, "memcpyAsync: only device-to-device copies can be recorded into a graph");
  HIP_CHECK(hipMemcpyAsync(dst, src, (size_t)size, kind, st));
  if (recorded) {
    ++*g_captureOpCalls;
    RecordedOp r;
    r.kind = RecordedOp::RAW;
    r.run = [dst, src, size](const RecordedOp&) { HIP_CHECK(hipMemcpyAsync(dst, src, (size_t)size, hipMemcpyDeviceToDevice, execStream())); };
    recordOp(std::move(r));
  }
  return 1;
  GUARD_END(0)
}
int memsetSync(Nd4jPointer dst, int value, Nd4jLong size, int, Nd4jPointer) {
  GUARD_BEGIN
  HIP_CHECK(hipMemset(dst, value, (size_t)size));
  return 1;
  GUARD_END(0)
}
int memsetAsync(Nd4jPointer dst, int value, Nd4jLong size, int, Nd4jPointer reserved) {
  GRAPH_BEGIN
  // a fill kernel rather than a memset node, so that callers may capture this call into a graph
  const hipStream_t st = streamOf(reserved);
  const bool recorded = rawOpInCapture(st);
  launchFill(st, dst, value, (size_t)size);
  if (recorded) {
    ++*g_captureOpCalls;
    RecordedOp r;
    r.kind = RecordedOp::RAW;
    r.run = [dst, value, size](const RecordedOp&) { launchFill(execStream(), dst, value, (size_t)size); };
    recordOp(std::move(r));
  }
  return 1;
  GUARD_END(0)
}

OpaqueLaunchContext defaultLaunchContext(void) {
  GUARD_BEGIN
  return static_cast<OpaqueLaunchContext>(LaunchContext::defaultContext());
  GUARD_END(nullptr)
}
Nd4jPointer lcScalarPointer(OpaqueLaunchContext lc) { return lc ? lc->scalarBuffer : nullptr; }
Nd4jPointer lcReductionPointer(OpaqueLaunchContext lc) { return lc ? lc->reductionBuffer : nullptr; }
Nd4jPointer lcAllocationPointer(OpaqueLaunchContext lc) { return lc ? lc->allocationBuffer : nullptr; }
Nd4jPointer lcExecutionStream(OpaqueLaunchContext lc) { return lc ? &lc->execStream : nullptr; }
Nd4jPointer lcCopyStream(OpaqueLaunchContext lc) { return lc ? &lc->copyStream : nullptr; }
Nd4jPointer lcBlasHandle(OpaqueLaunchContext) { return nullptr; }
Nd4jPointer lcSolverHandle(OpaqueLaunchContext) { return nullptr; }
Nd4jPointer lcScalarPointerPtr(OpaqueLaunchContext* lc) { return lc ? lcScalarPointer(*lc) : nullptr; }
Nd4jPointer lcReductionPointerPtr(OpaqueLaunchContext* lc) { return lc ? lcReductionPointer(*lc) : nullptr; }
Nd4jPointer lcAllocationPointerPtr(OpaqueLaunchContext* lc) { return lc ? lcAllocationPointer(*lc) : nullptr; }
Nd4jPointer lcExecutionStreamPtr(OpaqueLaunchContext* lc) { return lc ? lcExecutionStream(*lc) : nullptr; }
Nd4jPointer lcCopyStreamPtr(OpaqueLaunchContext* lc) { return lc ? lcCopyStream(*lc) : nullptr; }
Nd4jPointer lcBlasHandlePtr(OpaqueLaunchContext*) { return nullptr; }

// ---- start-up queries of a device backend ---------------------------------------------------------------------------
// Peer access between devices (legacy/cuda/NativeOps.cu:1015-1095): supported when every device reaches every other,
// and trivially with one device.
static bool g_supportedP2P = false, g_allowedP2P = false;
void checkP2P(void) {
  int n = 0, cur = 0;
  if (hipGetDeviceCount(&n) != hipSuccess) { (void)hipGetLastError(); n = 0; }
  bool all = true;
  if (n > 1) {
    (void)hipGetDevice(&cur);
    for (int a = 0; a < n && all; a++)
      for (int b = 0; b < n; b++) {
        if (a == b) continue;
        int can = 0;
        if (hipDeviceCanAccessPeer(&can, a, b) != hipSuccess) { (void)hipGetLastError(); can = 0; }
        if (!can) { all = false; break; }
      }
  }
  g_supportedP2P = all;
}
void enableP2P(bool enable) {
  if (enable == g_allowedP2P) return;
  int n = 0, cur = 0;
  if (hipGetDeviceCount(&n) != hipSuccess) { (void)hipGetLastError(); n = 0; }
  if (n > 1) {
    (void)hipGetDevice(&cur);
    for (int a = 0; a < n; a++)
      for (int b = 0; b < n; b++) {
        if (a == b) continue;
        int can = 0;
        (void)hipSetDevice(a);
        if (hipDeviceCanAccessPeer(&can, a, b) != hipSuccess) can = 0;
        if (can) { if (enable) (void)hipDeviceEnablePeerAccess(b, 0); else (void)hipDeviceDisablePeerAccess(b); }
        (void)hipGetLastError();   // "already enabled" and the like are not failures of this call
      }
    (void)hipSetDevice(cur);
  }
  g_allowedP2P = enable;
}
bool isP2PAvailable(void) {
  static std::once_flag once;
  std::call_once(once, [] { checkP2P(); });   // the reference's initializeDevicesAndFunctions runs the check
  return g_supportedP2P;
}
void initializeFunctions(Nd4jPointer*) {}     // the host BLAS function table of the CPU backend; nothing here calls a vendor BLAS
bool isBlasVersionMatches(int, int, int) { return true; }
int binaryLevel(void) { return 0; }           // legacy/cuda/NativeOps.cu:2769-2775
int optimalLevel(void) { return 0; }
bool isMinimalRequirementsMet(void) { return true; }
bool isOptimalRequirementsMet(void) { return true; }
bool isExperimentalEnabled(void) { return false; }
void setOmpMinThreads(int) {}
void setGridLimit(int) {}
Nd4jPointer getConstantSpace(void) { return nullptr; }

// ---- outside this backend's path --------------------------------------------------------------------------------------
static void notImplemented(const char* fn) { errorRef().set(1, std::string(fn) + " is not implemented in nd4j-hip"); }
void execRandom(Nd4jPointer*, int, Nd4jPointer, OpaqueNDArray, void*) { notImplemented("execRandom"); }
void execRandom2(Nd4jPointer*, int, Nd4jPointer, OpaqueNDArray, OpaqueNDArray, void*) { notImplemented("execRandom2"); }
void execRandom3(Nd4jPointer*, int, Nd4jPointer, OpaqueNDArray, OpaqueNDArray, OpaqueNDArray, void*) { notImplemented("execRandom3"); }
void sort(Nd4jPointer*, OpaqueNDArray, bool) { notImplemented("sort"); }
void sortTad(Nd4jPointer*, OpaqueNDArray, Nd4jLong*, Nd4jLong, Nd4jLong*, Nd4jLong*, bool) { notImplemented("sortTad"); }
void shuffle(Nd4jPointer*, OpaqueNDArrayArr, OpaqueNDArrayArr, int, OpaqueNDArray, OpaqueNDArray) { notImplemented("shuffle"); }
void pullRows(Nd4jPointer*, OpaqueNDArray, OpaqueNDArray, Nd4jLong, OpaqueNDArray, Nd4jLong) { notImplemented("pullRows"); }
void convertTypes(Nd4jPointer*, int, Nd4jPointer, Nd4jLong, int, Nd4jPointer) { notImplemented("convertTypes"); }

// ---- data buffers -----------------------------------------------------------------------------------
OpaqueDataBuffer* allocateDataBuffer(Nd4jLong elements, int dataType, bool allocateBoth) {
  GUARD_BEGIN
  DataType dt = (DataType)dataType;
  ND4J_REQUIRE(sizeOf(dt) > 0, "allocateDataBuffer: unsupported data type " + std::to_string(dataType));
  ND4J_REQUIRE(elements >= 0, "allocateDataBuffer: negative length");
  // zero elements still owns one element, as in the reference (NativeOpsHelpers_DataBuffers.cpp allocateDataBuffer)
  size_t bytes = (size_t)(elements == 0 ? 1 : elements) * sizeOf(dt);
  auto* h = new Nd4jHipDataBuffer();
  h->db = std::make_shared<DataBuffer>(bytes, dt, allocateBoth);
  return h;
  GUARD_END(nullptr)
}
OpaqueDataBuffer* dbAllocateDataBuffer(Nd4jLong elements, int dataType, bool allocateBoth) {
  return allocateDataBuffer(elements, dataType, allocateBoth);
}
OpaqueDataBuffer* dbCreateExternalDataBuffer(Nd4jLong elements, int dataType, Nd4jPointer primary, Nd4jPointer special) {
  GUARD_BEGIN
  DataType dt = (DataType)dataType;
  ND4J_REQUIRE(sizeOf(dt) > 0, "dbCreateExternalDataBuffer: unsupported data type");
  auto* h = new Nd4jHipDataBuffer();
  h->db = std::make_shared<DataBuffer>(primary, special, (size_t)elements * sizeOf(dt), dt);
  return h;
  GUARD_END(nullptr)
}
OpaqueDataBuffer* dbCreateView(OpaqueDataBuffer* dataBuffer, Nd4jLong length) {
  GUARD_BEGIN
  ND4J_REQUIRE(dataBuffer && dataBuffer->db, "dbCreateView: buffer is null");
  auto* h = new Nd4jHipDataBuffer();
  h->db = dataBuffer->db;
  h->offsetBytes = dataBuffer->offsetBytes;
  (void)length;
  return h;
  GUARD_END(nullptr)
}
Nd4jPointer dbPrimaryBuffer(OpaqueDataBuffer* b) { return b ? b->primary() : nullptr; }
Nd4jPointer dbSpecialBuffer(OpaqueDataBuffer* b) { return b ? b->special() : nullptr; }
Nd4jLong dbBufferLength(OpaqueDataBuffer* b) { return b && b->db ? b->db->numElements() : 0; }
void dbSetPrimaryBuffer(OpaqueDataBuffer* b, Nd4jPointer p, Nd4jLong numBytes) {
  GUARD_BEGIN
  ND4J_REQUIRE(b && b->db, "dbSetPrimaryBuffer: buffer is null");
  b->db->releasePrimary();
  b->db->primary = p; b->db->ownsPrimary = false; b->db->lenBytes = (size_t)numBytes;
  b->db->tickWritePrimary();
  GUARD_END_VOID
}
void dbSetSpecialBuffer(OpaqueDataBuffer* b, Nd4jPointer p, Nd4jLong numBytes) {
  GUARD_BEGIN
  ND4J_REQUIRE(b && b->db, "dbSetSpecialBuffer: buffer is null");
  if (b->db->ownsSpecial && b->db->special) HIP_CHECK(hipFree(b->db->special));
  b->db->special = p; b->db->ownsSpecial = false; b->db->lenBytes = (size_t)numBytes;
  b->db->tickWriteSpecial();
  GUARD_END_VOID
}
void dbAllocatePrimaryBuffer(OpaqueDataBuffer* b) {
  GUARD_BEGIN
  ND4J_REQUIRE(b && b->db, "dbAllocatePrimaryBuffer: buffer is null");
  b->db->allocatePrimary();
  GUARD_END_VOID
}
void dbAllocateSpecialBuffer(OpaqueDataBuffer* b) {
  GUARD_BEGIN
  ND4J_REQUIRE(b && b->db, "dbAllocateSpecialBuffer: buffer is null");
  b->db->allocateSpecial();
  GUARD_END_VOID
}
void dbExpandBuffer(OpaqueDataBuffer* b, Nd4jLong elements) {
  GUARD_BEGIN
  ND4J_REQUIRE(b && b->db, "dbExpandBuffer: buffer is null");
  b->db->expand((size_t)elements * sizeOf(b->db->dtype));
  GUARD_END_VOID
}
void dbExpand(OpaqueDataBuffer* b, Nd4jLong elements) { dbExpandBuffer(b, elements); }
int dbUseCount(OpaqueDataBuffer* b) { return b && b->db ? (int)b->db.use_count() : 0; }
void dbSyncToSpecial(OpaqueDataBuffer* b) {
  GUARD_BEGIN
  ND4J_REQUIRE(b && b->db, "dbSyncToSpecial: buffer is null");
  b->db->syncToSpecial();
  GUARD_END_VOID
}
void dbSyncToPrimary(OpaqueDataBuffer* b) {
  GUARD_BEGIN
  ND4J_REQUIRE(b && b->db, "dbSyncToPrimary: buffer is null");
  b->db->syncToPrimary();
  GUARD_END_VOID
}
void dbTickHostRead(OpaqueDataBuffer* b) { if (b && b->db) b->db->tickReadPrimary(); }
void dbTickHostWrite(OpaqueDataBuffer* b) { if (b && b->db) b->db->tickWritePrimary(); }
void dbTickDeviceRead(OpaqueDataBuffer* b) { if (b && b->db) b->db->tickReadSpecial(); }
void dbTickDeviceWrite(OpaqueDataBuffer* b) { if (b && b->db) b->db->tickWriteSpecial(); }
void dbClose(OpaqueDataBuffer* b) {
  GUARD_BEGIN
  if (b && b->db) b->db->close();
  GUARD_END_VOID
}
int dbDeviceId(OpaqueDataBuffer* b) { return b && b->db ? b->db->deviceId : 0; }
void dbSetDeviceId(OpaqueDataBuffer* b, int deviceId) { if (b && b->db) b->db->deviceId = deviceId; }
int dbLocality(OpaqueDataBuffer* b) {
  if (!b || !b->db) return 0;
  bool p = b->db->isPrimaryActual(), s = b->db->isSpecialActual();
  if (p && !s) return -1;
  if (s && !p) return 1;
  return 0;
}
void deleteDataBuffer(OpaqueDataBuffer* b) { delete b; }

// ---- shape descriptors --------------------------------------------------------------------------------
OpaqueConstantShapeBuffer shapeBufferEx(int rank, Nd4jLong* shp, Nd4jLong* strides, int dtype, char order, Nd4jLong ews, Nd4jLong extras) {
  GUARD_BEGIN
  ND4J_REQUIRE(rank >= 0 && rank <= MAX_RANK, "shapeBuffer: rank out of range");
  ND4J_REQUIRE(rank == 0 || shp != nullptr, "shapeBuffer: shape is null");
  std::vector<LongType> s(shp, shp + rank);
  auto si = makeShapeInfo((DataType)dtype, order, s, strides, extras);
  (void)ews;  // recomputed from the strides
  return static_cast<OpaqueConstantShapeBuffer>(cachedShapeBuffer(si.data()));
  GUARD_END(nullptr)
}
OpaqueConstantShapeBuffer shapeBuffer(int rank, Nd4jLong* shp, Nd4jLong* strides, int dtype, char order, Nd4jLong ews, bool empty) {
  return shapeBufferEx(rank, shp, strides, dtype, order, ews, empty ? ARRAY_EMPTY : 0);
}
OpaqueConstantShapeBuffer cacheAndStoreShapeBuffer(Nd4jLong* shapeInfo) {
  GUARD_BEGIN
  return static_cast<OpaqueConstantShapeBuffer>(cachedShapeBuffer(shapeInfo));
  GUARD_END(nullptr)
}
Nd4jPointer getConstantShapeBufferPrimary(OpaqueConstantShapeBuffer b) { return b ? (Nd4jPointer)b->primary() : nullptr; }
Nd4jPointer getConstantShapeBufferSpecial(OpaqueConstantShapeBuffer b) {
  GUARD_BEGIN
  return b ? (Nd4jPointer)b->special() : nullptr;
  GUARD_END(nullptr)
}
void deleteConstantShapeBuffer(OpaqueConstantShapeBuffer*) {}

// ---- array handles ------------------------------------------------------------------------------------
OpaqueNDArray createOpaqueNDArray(OpaqueDataBuffer* shapeInfo, OpaqueDataBuffer* buffer, OpaqueDataBuffer* specialBuffer, Nd4jLong offset) {
  GUARD_BEGIN
  ND4J_REQUIRE(shapeInfo != nullptr, "createOpaqueNDArray: Shape info was null!");
  const LongType* si = reinterpret_cast<const LongType*>(shapeInfo->primary());
  ND4J_REQUIRE(si != nullptr, "createOpaqueNDArray: shapeInfo->primary() returned nullptr - shape buffer is invalid!");
  const int rank = shape::rank(si);
  ND4J_REQUIRE(rank >= 0 && rank <= MAX_RANK, "createOpaqueNDArray: rank out of range");
  if (shape::isEmpty(si) && buffer != nullptr) ND4J_THROW("createOpaqueNDArray: Shape info was empty but buffer was not null!");
  if (!shape::isEmpty(si) && buffer == nullptr) ND4J_THROW("createOpaqueNDArray: Shape info was not empty but buffer was null!");
  ND4J_REQUIRE(shape::dataType(si) != UNKNOWN, "createOpaqueNDArray: descriptor carries no known data type");
  (void)specialBuffer;  // the device side lives in the same buffer object
  auto* a = new Nd4jHipNDArray();
  a->si.assign(si, si + shape::shapeInfoLength(rank));
  a->offset = offset;
  if (buffer) {
    a->buf = buffer->db;
    a->bufOffsetBytes = buffer->offsetBytes;
    // bounds: the furthest element of the view must lie inside the buffer
    LongType maxOff = offset;
    for (int d = 0; d < rank; d++) {
      LongType st = shape::strideOf(si)[d];
      if (shape::shapeOf(si)[d] > 0 && st > 0) maxOff += (shape::shapeOf(si)[d] - 1) * st;
    }
    ND4J_REQUIRE(offset >= 0, "createOpaqueNDArray: negative offset");
    ND4J_REQUIRE((size_t)(maxOff + 1) * sizeOf(a->dataType()) + a->bufOffsetBytes <= a->buf->lenBytes,
                 "createOpaqueNDArray: shape/strides/offset reach beyond the end of the data buffer");
  }
  return a;
  GUARD_END(nullptr)
}
void deleteNDArray(OpaqueNDArray array) { delete array; }
Nd4jLong getOpaqueNDArrayOffset(OpaqueNDArray a) { return a ? a->offset : 0; }
const Nd4jLong* getOpaqueNDArrayShapeInfo(OpaqueNDArray a) { return a ? a->shapeInfo() : nullptr; }
void* getOpaqueNDArrayBuffer(OpaqueNDArray a) { return a ? a->buffer() : nullptr; }
void* getOpaqueNDArraySpecialBuffer(OpaqueNDArray a) { return a ? a->specialBuffer() : nullptr; }
Nd4jLong getOpaqueNDArrayLength(OpaqueNDArray a) { return a && a->buf ? a->buf->numElements() : 0; }
Nd4jLong getOpaqueNDArrayShapeInfoLength(OpaqueNDArray a) { return a ? shape::shapeInfoLength(a->rankOf()) : 0; }

// ---- TAD packs -------------------------------------------------------------------------------------------
OpaqueTadPack* tadOnlyShapeInfo(OpaqueDataBuffer* hXShapeInfo, Nd4jLong* dimension, Nd4jLong dimensionLength) {
  GUARD_BEGIN
  ND4J_REQUIRE(hXShapeInfo && hXShapeInfo->primary(), "tadOnlyShapeInfo: shape info is null");
  return static_cast<OpaqueTadPack*>(tadForDimensions(reinterpret_cast<const LongType*>(hXShapeInfo->primary()), dimension, (int)dimensionLength));
  GUARD_END(nullptr)
}
const Nd4jLong* getPrimaryShapeInfo(OpaqueTadPack* p) { return p ? p->tadShape->primary() : nullptr; }
const Nd4jLong* getPrimaryOffsets(OpaqueTadPack* p) { return p ? p->offsets.data() : nullptr; }
const Nd4jLong* getSpecialShapeInfo(OpaqueTadPack* p) {
  GUARD_BEGIN
  return p ? p->tadShape->special() : nullptr;
  GUARD_END(nullptr)
}
const Nd4jLong* getSpecialOffsets(OpaqueTadPack* p) {
  GUARD_BEGIN
  return p ? p->specialOffsets() : nullptr;
  GUARD_END(nullptr)
}
Nd4jLong getNumberOfTads(OpaqueTadPack* p) { return p ? p->numTads : 0; }
int getShapeInfoLength(OpaqueTadPack* p) { return p ? shape::shapeInfoLength(shape::rank(p->tadShape->primary())) : 0; }
void deleteTadPack(OpaqueTadPack*) {}

// ---- legacy loops --------------------------------------------------------------------------------------------
static void runUnary(const char* fn, UnaryKind k, NDArray* x, NDArray* z) {
  if (x->isEmpty() || z->isEmpty()) return;
  EwPlan p = buildEwPlan({z->shapeInfo(), x->shapeInfo()});
  prepareSpecialUse({z}, {x});
  launchUnary(execStream(), k, x->dataType(), z->dataType(), x->specialBuffer(), z->specialBuffer(), p);
  registerSpecialUse({z}, {x});
}

// n extra parameters, held in data type dt (the executioner converts an op's extraArgs to the array's type before the call);
// the pointer may be device or host memory, so they are fetched with a blocking copy
static std::vector<double> fetchParams(const char* fn, const void* extraParams, DataType dt, int n) {
  if (extraParams == nullptr) ND4J_THROW(std::string(fn) + ": this op reads " + std::to_string(n) + " extra parameters, got none");
  unsigned char raw[64];
  const size_t w = sizeOf(dt);
  ND4J_REQUIRE(w > 0 && w * n <= sizeof(raw), std::string(fn) + ": unsupported type of the extra parameters");
  ND4J_REQUIRE(!captureActive(), std::string(fn) + ": ops that read extra parameters cannot be recorded into a graph (the parameters are fetched with a blocking copy)");
  HIP_CHECK(hipStreamSynchronize(execStream()));
  HIP_CHECK(hipMemcpy(raw, extraParams, n * w, hipMemcpyDefault));
  std::vector<double> out(n);
  for (int i = 0; i < n; i++) {
    const void* p = raw + i * w;
    switch (dt) {
      case INT32: out[i] = *(const int*)p; break;
      case INT64: out[i] = (double)*(const LongType*)p; break;
      case BOOL: out[i] = *(const unsigned char*)p; break;
      default: out[i] = hostValueAsDouble(p, dt);
    }
  }
  return out;
}
// [compare, eps, mode] (MatchCondition family) or [compare, set, eps, mode] (the CompareAndSet family)
static CondParams condParams(const char* fn, const void* extraParams, DataType dt, bool withSet) {
  auto v = fetchParams(fn, extraParams, dt, withSet ? 4 : 3);
  CondParams c;
  c.compare = v[0];
  c.set = withSet ? v[1] : 0.0;
  c.eps = v[withSet ? 2 : 1];
  c.mode = (int)v[withSet ? 3 : 2];
  c.xdt = (int)dt;
  ND4J_REQUIRE(c.mode >= 0 && c.mode <= 15, std::string(fn) + ": undefined match condition " + std::to_string(c.mode));
  return c;
}

// The transforms that read two extra parameters.  extraParams holds them in the array's own type (the executioner
// converts its extraArgs to X before the call); it may be device or host memory, so they are fetched with a blocking copy.
static void runUnaryWithParams(const char* fn, Scalar2Kind k, NDArray* x, NDArray* z, const void* extraParams) {
  const int nParams = k == S2_STABILIZE ? 1 : 2;
  if (extraParams == nullptr) ND4J_THROW(std::string(fn) + (nParams == 1 ? ": this op needs one extra parameter" : ": this op needs two extra parameters"));
  if (x->isEmpty() || z->isEmpty()) return;
  unsigned char raw[16];
  const size_t w = sizeOf(x->dataType());
  HIP_CHECK(hipStreamSynchronize(execStream()));
  HIP_CHECK(hipMemcpy(raw, extraParams, nParams * w, hipMemcpyDefault));
  const double s1 = hostValueAsDouble(raw, x->dataType()), s2 = nParams > 1 ? hostValueAsDouble(raw + w, x->dataType()) : 0.0;
  EwPlan p = buildEwPlan({z->shapeInfo(), x->shapeInfo()});
  prepareSpecialUse({z}, {x});
  launchScalar2Op(execStream(), k, x->dataType(), z->dataType(), x->specialBuffer(), s1, s2, z->specialBuffer(), p);
  registerSpecialUse({z}, {x});
}

void execTransformStrict(Nd4jPointer* extraPointers, int opNum, OpaqueNDArray xa, void* extraParams, OpaqueNDArray za) {
  OP_BEGIN(callerStream(extraPointers))
  NDArray* x = arr(xa, "execTransformStrict", "x"); NDArray* z = arr(za, "execTransformStrict", "z");
  transformStrictImpl(opNum, x, extraParams, z);
  if (captureActive() && !(opNum == 2 || opNum == 3 || opNum == 19 || opNum == 25)) {
    RecordedOp r;
    r.kind = RecordedOp::TRANSFORM_STRICT; r.opNum = opNum; r.x = x; r.z = z;
    r.run = [](const RecordedOp& o) { transformStrictImpl(o.opNum, o.x, nullptr, o.z); };
    recordOp(std::move(r));
  }
  GUARD_END_VOID
}
}  // extern "C"
static void transformStrictImpl(int opNum, NDArray* x, void* extraParams, NDArray* z) {
  {
  // X -> X over float types only (NativeOpExecutioner_transform.cpp:115-131)
  ND4J_REQUIRE(x->dataType() == z->dataType() && isFloatType(x->dataType()),
               std::string("NativeOpExecutioner::execTransformStrict requires X & Z to have same floating point type, got ") + dtypeName(x->dataType()) + " and " + dtypeName(z->dataType()));
  if (opNum == 2 || opNum == 3 || opNum == 19 || opNum == 25) {   // ScaledTanh, Affine, Stabilize, SetRange (loops/legacy_ops.h:54-60)
    runUnaryWithParams("execTransformStrict", opNum == 2 ? S2_SCALED_TANH : opNum == 3 ? S2_AFFINE : opNum == 19 ? S2_STABILIZE : S2_SET_RANGE, x, z, extraParams);
    return;
  }
  UnaryKind k;
  switch (opNum) {  // loops/legacy_ops.h:54-64
    case 22: k = U_COS; break; case 23: k = U_EXP; break; case 24: k = U_LOG; break; case 26: k = U_SIGMOID; break;
    case 27: k = U_SIN; break; case 28: k = U_SOFTPLUS; break; case 29: k = U_TANH; break; case 43: k = U_SWISH; break;
    case 45: k = U_ERF; break; case 53: k = U_GELU; break; case 55: k = U_PRECISE_GELU; break;
    case 4: k = U_TANH_D; break; case 6: k = U_SIGMOID_D; break; case 7: k = U_SOFTSIGN_D; break; case 8: k = U_TAN_D; break;
    case 9: k = U_SELU_D; break; case 11: k = U_RATIONAL_TANH_D; break; case 12: k = U_RECTIFIED_TANH_D; break;
    case 13: k = U_SWISH_D; break; case 14: k = U_ACOSH_D; break; case 15: k = U_ASINH_D; break; case 16: k = U_SINH_D; break;
    case 17: k = U_LOG_SIGMOID_D; break; case 18: k = U_SPECIAL_D; break; case 21: k = U_CUBE_D; break;
    case 30: k = U_ACOS; break; case 31: k = U_ASIN; break; case 32: k = U_ATAN; break; case 33: k = U_HARD_TANH; break;
    case 34: k = U_SOFTSIGN; break; case 36: k = U_HARD_SIGMOID; break; case 37: k = U_RATIONAL_TANH; break;
    case 38: k = U_RECTIFIED_TANH; break; case 39: k = U_SINH; break; case 40: k = U_COSH; break; case 41: k = U_TAN; break;
    case 42: k = U_SELU; break; case 44: k = U_LOG1P; break; case 46: k = U_ACOSH; break; case 47: k = U_ASINH; break;
    case 48: k = U_RINT; break; case 49: k = U_LOG_SIGMOID; break; case 50: k = U_ERFC; break; case 51: k = U_EXPM1; break;
    case 52: k = U_ATANH; break; case 54: k = U_GELU_D; break; case 56: k = U_PRECISE_GELU_D; break; case 57: k = U_MISH; break;
    case 58: k = U_MISH_D; break;
    // 5 HardTanhDerivative and 10 HardSigmoidDerivative: the reference declares them through a macro that takes the
    // derivative's expression as its CONDITION and the input as both outcomes (ops/ops.h:222-226 through
    // ops/op_macros_unary.h:109-113), so both return the input unchanged; restated as they compute
    case 5: case 10: k = U_IDENTITY; break;
    case 20: k = U_STABILIZE_FP16; break;   // ops/ops.h:381-384
    default: ND4J_THROW("execTransformStrict: opNum " + std::to_string(opNum) + " is not implemented in nd4j-hip");
  }
  runUnary("execTransformStrict", k, x, z);
  }
}
extern "C" {
void execTransformFloat(Nd4jPointer* extraPointers, int opNum, OpaqueNDArray xa, void*, OpaqueNDArray za) {
  OP_BEGIN(callerStream(extraPointers))
  NDArray* x = arr(xa, "execTransformFloat", "x"); NDArray* z = arr(za, "execTransformFloat", "z");
  ND4J_REQUIRE(isFloatType(z->dataType()), "NativeOpExecutioner::execTransformFloat requires Z to have floating point type");
  // any common type into any float type (NativeOpExecutioner_transform.cpp:35-37: SD_COMMON_TYPES x SD_FLOAT_TYPES); an
  // integer or bool element is converted to Z first and the op runs in Z's arithmetic
  ND4J_REQUIRE(isFloatType(x->dataType()) || x->dataType() == INT32 || x->dataType() == INT64 || x->dataType() == BOOL,
               std::string("execTransformFloat: input type ") + dtypeName(x->dataType()) + " is not implemented in nd4j-hip");
  UnaryKind k;
  switch (opNum) {  // loops/legacy_ops.h:67
    case 1: k = U_SQRT; break; case 3: k = U_RSQRT; break;
    default: ND4J_THROW("execTransformFloat: opNum " + std::to_string(opNum) + " is not implemented in nd4j-hip");
  }
  runUnary("execTransformFloat", k, x, z);
  GUARD_END_VOID
}
void execTransformSame(Nd4jPointer* extraPointers, int opNum, OpaqueNDArray xa, void* extraParams, OpaqueNDArray za) {
  OP_BEGIN(callerStream(extraPointers))
  NDArray* x = arr(xa, "execTransformSame", "x"); NDArray* z = arr(za, "execTransformSame", "z");
  ND4J_REQUIRE(x->dataType() == z->dataType(), "NativeOpExecutioner::execTransformSame requires X & Z to have same type");
  ND4J_REQUIRE(isFloatType(x->dataType()) || isIntLike(x->dataType()), "execTransformSame: this data type is not implemented in nd4j-hip");
  if (opNum == 19) {
    ND4J_REQUIRE(isFloatType(x->dataType()), "execTransformSame: ClipByValue on integer arrays is not implemented in nd4j-hip");   // ClipByValue (loops/legacy_ops.h:43)
    runUnaryWithParams("execTransformSame", S2_CLIP_BY_VALUE, x, z, extraParams);
    return;
  }
  if (opNum == 13) {   // CompareAndSetTransform (loops/legacy_ops.h:42)
    ND4J_REQUIRE(isFloatType(x->dataType()) || x->dataType() == INT32, "execTransformSame: CompareAndSetTransform takes float or INT32 arrays here");
    if (x->isEmpty() || z->isEmpty()) return;
    const CondParams c = condParams("execTransformSame", extraParams, x->dataType(), true);
    EwPlan p = buildEwPlan({z->shapeInfo(), x->shapeInfo()});
    prepareSpecialUse({z}, {x});
    launchCondElementwise(execStream(), C_SET_TRANSFORM, c, x->dataType(), z->dataType(), x->specialBuffer(), nullptr, z->specialBuffer(), p, 0.0, false);
    registerSpecialUse({z}, {x});
    return;
  }
  UnaryKind k;
  switch (opNum) {  // loops/legacy_ops.h:40-44
    case 0: k = U_ABS; break; case 3: k = U_NEG; break; case 6: k = U_CUBE; break; case 7: k = U_ONE_MINUS; break;
    case 11: k = U_RECIPROCAL; break; case 12: k = U_SQUARE; break; case 15: case 21: k = U_IDENTITY; break;
    case 2: k = U_ONES; break; case 4: k = U_ROUND; break; case 5: k = U_TIMES_ONE_MINUS; break; case 17: k = U_CEIL; break;
    case 18: k = U_FLOOR; break;
    case 1: k = U_SIGN_REF; break;   // Sign as the reference computes it (ops/ops.h:217-219): 1 for every non-zero number, -1 for 0 and NaN
    default: ND4J_THROW("execTransformSame: opNum " + std::to_string(opNum) + " is not implemented in nd4j-hip");
  }
  runUnary("execTransformSame", k, x, z);
  GUARD_END_VOID
}
void execTransformAny(Nd4jPointer* extraPointers, int opNum, OpaqueNDArray xa, void*, OpaqueNDArray za) {
  OP_BEGIN(callerStream(extraPointers))
  NDArray* x = arr(xa, "execTransformAny", "x"); NDArray* z = arr(za, "execTransformAny", "z");
  ND4J_REQUIRE(opNum == 0, "execTransformAny: only Assign (opNum 0) exists (loops/legacy_ops.h:46)");
  runUnary("execTransformAny", U_IDENTITY, x, z);
  if (captureActive()) {
    RecordedOp r;
    r.kind = RecordedOp::TRANSFORM_ANY; r.opNum = 0; r.x = x; r.z = z;
    r.run = [](const RecordedOp& o) { runUnary("execTransformAny", U_IDENTITY, o.x, o.z); };
    recordOp(std::move(r));
  }
  GUARD_END_VOID
}

static PairwiseKind pairwiseKind(int opNum) {
  switch (opNum) {  // loops/legacy_ops.h:121-129
    case 0: return P_ADD; case 1: return P_COPY; case 2: return P_DIV; case 3: return P_MUL; case 5: return P_RSUB;
    case 6: return P_SUB; case 7: return P_MAX; case 8: return P_MIN; case 11: return P_RDIV; case 20: return P_SQSUB;
    case 4: return P_POW; case 9: return P_COPY; case 14: return P_REMAINDER; case 15: return P_FMOD; case 16: return P_ATAN2;
    case 17: return P_TRUNCATE_DIV; case 18: return P_FLOOR_DIV; case 19: return P_FLOOR_MOD; case 21: return P_REVERSE_MOD;
    case 22: return P_SAFE_DIVIDE; case 23: return P_MOD; case 27: return P_LOGICAL_OR; case 28: return P_LOGICAL_XOR;
    case 29: return P_LOGICAL_NOT; case 30: return P_LOGICAL_AND; case 34: return P_AMAX; case 35: return P_AMIN;
    case 36: return P_TRUNCATE_MOD; case 37: return P_REPLACE_NANS; case 38: return P_DIVIDE_NO_NAN;
    case 24: return P_REL_ERR; case 31: return P_POW_DERIV; case 32: return P_LOG_POISSON; case 33: return P_LOG_POISSON_FULL;
    case 39: return P_IGAMMA; case 40: return P_IGAMMAC;
    // 10 Axpy, 12/13 CompareAndSet / CompareAndReplace and 25/26 the thresholded relative errors read extraParams and are
    // served before this table is consulted
    default: ND4J_THROW("execPairwiseTransform: opNum " + std::to_string(opNum) + " is not implemented in nd4j-hip");
  }
}
void execPairwiseTransform(Nd4jPointer* extraPointers, int opNum, OpaqueNDArray xa, OpaqueNDArray ya, OpaqueNDArray za, void* extraParams) {
  OP_BEGIN(callerStream(extraPointers))
  NDArray* x = arr(xa, "execPairwiseTransform", "x"); NDArray* y = arr(ya, "execPairwiseTransform", "y");
  NDArray* z = arr(za, "execPairwiseTransform", "z");
  if (opNum == 12 || opNum == 13) {   // CompareAndSet, CompareAndReplace (loops/legacy_ops.h:123): parameters in Z's type
    // values travel through a double on the way to Z, which INT64 does not survive beyond 2^53
    ND4J_REQUIRE((isFloatType(z->dataType()) || z->dataType() == INT32) && x->dataType() == z->dataType() && y->dataType() == z->dataType(), "execPairwiseTransform: CompareAndSet / CompareAndReplace take float or INT32 arrays of one type here");
    if (z->isEmpty()) return;
    const CondParams c = condParams("execPairwiseTransform", extraParams, z->dataType(), true);
    EwPlan p = buildEwPlan({z->shapeInfo(), x->shapeInfo(), y->shapeInfo()});
    prepareSpecialUse({z}, {x, y});
    launchCondElementwise(execStream(), opNum == 12 ? C_SET : C_REPLACE, c, y->dataType(), z->dataType(), x->specialBuffer(), y->specialBuffer(), z->specialBuffer(), p, 0.0, false);
    registerSpecialUse({z}, {x, y});
    return;
  }
  if (opNum == 10 || opNum == 25 || opNum == 26) {   // Axpy [alpha], BinaryRelativeError [threshold], BinaryMinimumAbsoluteRelativeError [rel, abs]
    ND4J_REQUIRE(isFloatType(z->dataType()) && x->dataType() == z->dataType() && y->dataType() == z->dataType(), "execPairwiseTransform: Axpy and the thresholded relative errors take float arrays of one type here");
    if (z->isEmpty()) return;
    const auto v = fetchParams("execPairwiseTransform", extraParams, z->dataType(), opNum == 26 ? 2 : 1);
    CondParams c;
    c.compare = v[0]; c.set = opNum == 26 ? v[1] : 0.0; c.eps = 0.0; c.mode = 0; c.xdt = (int)z->dataType();
    EwPlan p = buildEwPlan({z->shapeInfo(), x->shapeInfo(), y->shapeInfo()});
    prepareSpecialUse({z}, {x, y});
    launchCondElementwise(execStream(), opNum == 10 ? C_AXPY : opNum == 25 ? C_BIN_REL_ERR : C_BIN_MIN_ABS_REL_ERR, c, y->dataType(), z->dataType(), x->specialBuffer(),
                          y->specialBuffer(), z->specialBuffer(), p, 0.0, false);
    registerSpecialUse({z}, {x, y});
    return;
  }
  pairwiseImpl(opNum, x, y, z);
  if (captureActive()) {
    RecordedOp r;
    r.kind = RecordedOp::PAIRWISE; r.opNum = opNum; r.x = x; r.y = y; r.z = z;
    r.run = [](const RecordedOp& o) { pairwiseImpl(o.opNum, o.x, o.y, o.z); };
    recordOp(std::move(r));
  }
  GUARD_END_VOID
}
}  // extern "C"
static void pairwiseImpl(int opNum, NDArray* x, NDArray* y, NDArray* z) {
  // NativeOpExecutioner_pairwise_floats.cpp:34-57
  ND4J_REQUIRE(x->dataType() == z->dataType() || y->dataType() == z->dataType(),
               std::string("NativeOpExecutioner::execPairwiseTransform requires X or Y to have the same type as Z, got ") + dtypeName(x->dataType()) + ", " + dtypeName(y->dataType()) + " -> " + dtypeName(z->dataType()));
  {
    // all floating point, all integer / bool, or a floating point result from INT32 / INT64 / BOOL operands
    const bool allInt = isIntLike(x->dataType()) && isIntLike(y->dataType()) && isIntLike(z->dataType());
    auto loadable = [](DataType t) { return isFloatType(t) || t == INT32 || t == INT64 || t == BOOL; };
    ND4J_REQUIRE(allInt || (isFloatType(z->dataType()) && loadable(x->dataType()) && loadable(y->dataType())),
                 std::string("execPairwiseTransform: the combination ") + dtypeName(x->dataType()) + ", " + dtypeName(y->dataType()) + " -> " + dtypeName(z->dataType()) + " is not implemented in nd4j-hip");
  }
  PairwiseKind k = pairwiseKind(opNum);
  if (z->isEmpty()) return;
  EwPlan p = buildEwPlan({z->shapeInfo(), x->shapeInfo(), y->shapeInfo()});
  prepareSpecialUse({z}, {x, y});
  // each view's offset is applied once here (specialBuffer()); the reference's CPU facade adds x->offset()
  // a second time for views (legacy/cpu/NativeOps.cpp:1245-1257)
  launchPairwise(execStream(), k, x->dataType(), y->dataType(), z->dataType(), x->specialBuffer(), y->specialBuffer(), z->specialBuffer(), p);
  registerSpecialUse({z}, {x, y});
}
extern "C" {

static LongType hostScalarInt64(NDArray* s) {
  ND4J_REQUIRE(s->lengthOf() >= 1 && s->buf, "scalar operand is empty");
  s->buf->syncToPrimary();
  return *static_cast<const LongType*>(s->buffer());
}
static double hostScalar(NDArray* s) {
  ND4J_REQUIRE(s->lengthOf() >= 1 && s->buf, "scalar operand is empty");
  s->buf->syncToPrimary();
  const void* p = s->buffer();
  switch (s->dataType()) {
    case FLOAT32: return *(const float*)p;
    case DOUBLE: return *(const double*)p;
    case INT32: return *(const int*)p;
    case INT64: return (double)*(const LongType*)p;
    case BOOL: case UINT8: return *(const unsigned char*)p;
    case INT8: return *(const signed char*)p;
    case INT16: return *(const short*)p;
    case UINT16: return *(const unsigned short*)p;
    case UINT32: return *(const unsigned*)p;
    case UINT64: return (double)*(const unsigned long long*)p;
    case HALF: { unsigned short h = *(const unsigned short*)p; unsigned sign = (h & 0x8000u) << 16, e = (h >> 10) & 31, m = h & 1023; float f; unsigned u;
      if (e == 0) { f = (float)m / 16777216.0f; if (sign) f = -f; return f; }
      if (e == 31) u = sign | 0x7f800000u | (m << 13); else u = sign | ((e + 112) << 23) | (m << 13);
      memcpy(&f, &u, 4); return f; }
    case BFLOAT16: { unsigned u = ((unsigned)*(const unsigned short*)p) << 16; float f; memcpy(&f, &u, 4); return f; }
    default: ND4J_THROW("scalar operand has an unsupported data type");
  }
}
static PairwiseKind scalarKind(const char* fn, int opNum) {
  PairwiseKind k;
  switch (opNum) {  // loops/legacy_ops.h:78-86
    case 0: k = P_ADD; break; case 1: k = P_SUB; break; case 2: k = P_MUL; break; case 3: k = P_DIV; break;
    case 4: k = P_RDIV; break; case 5: k = P_RSUB; break; case 6: k = P_MAX; break; case 13: k = P_MIN; break; case 14: k = P_COPY; break;
    case 7: k = P_ELU; break; case 8: k = P_ELU_D; break; case 15: k = P_MOD; break; case 16: k = P_REVERSE_MOD; break;
    case 17: k = P_REMAINDER; break; case 18: k = P_FMOD; break; case 19: k = P_TRUNCATE_DIV; break; case 20: k = P_FLOOR_DIV; break;
    case 21: k = P_FLOOR_MOD; break; case 22: case 44: k = P_SQ_RSUB; break;   // (x - s)^2 == (s - x)^2
    case 23: k = P_SAFE_DIVIDE; break; case 24: k = P_AMAX; break; case 25: k = P_AMIN; break; case 26: k = P_ATAN2; break;
    case 27: k = P_LOGICAL_OR; break; case 28: k = P_LOGICAL_XOR; break; case 29: k = P_LOGICAL_NOT; break;
    case 30: k = P_LOGICAL_AND; break; case 31: k = P_POW; break; case 34: k = P_SXE_LOGITS_SMOOTHER; break;
    case 35: k = P_LEAKY_RELU; break; case 36: k = P_LEAKY_RELU_D; break; case 37: k = P_REPLACE_NANS; break;
    case 38: k = P_LOG_X; break; case 39: k = P_RELU; break; case 40: k = P_RELU6; break; case 41: k = P_STEP; break;
    case 42: k = P_LSTM_CLIP; break; case 43: k = P_TRUNCATE_MOD; break; case 45: k = P_REVERSE_POW; break;
    case 46: k = P_DIVIDE_NO_NAN; break; case 49: k = P_RELU_D; break;
    case 32: k = P_POW_DERIV; break; case 47: k = P_IGAMMA; break; case 48: k = P_IGAMMAC; break;   // 33 CompareAndSet is served above
    default: ND4J_THROW(std::string(fn) + ": opNum " + std::to_string(opNum) + " is not implemented in nd4j-hip");
  }
  return k;
}
void execScalar(Nd4jPointer* extraPointers, int opNum, OpaqueNDArray xa, OpaqueNDArray za, OpaqueNDArray sa, void* extraParams) {
  OP_BEGIN(callerStream(extraPointers))
  NDArray* x = arr(xa, "execScalar", "x"); NDArray* z = arr(za, "execScalar", "z"); NDArray* s = arr(sa, "execScalar", "scalar");
  ND4J_REQUIRE(x->dataType() == z->dataType() && (isFloatType(x->dataType()) || isIntLike(x->dataType())), "execScalar: nd4j-hip requires X and Z of one type");
  if (opNum == 33) {   // CompareAndSet with the scalar as second operand: z = cond(scalar) ? scalar : x (ops.h:719-840)
    ND4J_REQUIRE(isFloatType(x->dataType()) || x->dataType() == INT32, "execScalar: CompareAndSet takes float or INT32 arrays here");
    if (z->isEmpty()) return;
    const CondParams c = condParams("execScalar", extraParams, z->dataType(), true);
    const double sc = hostScalar(s);
    EwPlan p = buildEwPlan({z->shapeInfo(), x->shapeInfo()});
    prepareSpecialUse({z}, {x});
    launchCondElementwise(execStream(), C_SET, c, x->dataType(), z->dataType(), x->specialBuffer(), nullptr, z->specialBuffer(), p, sc, true);
    registerSpecialUse({z}, {x});
    return;
  }
  const PairwiseKind k = scalarKind("execScalar", opNum);
  if (z->isEmpty()) return;
  EwPlan p = buildEwPlan({z->shapeInfo(), x->shapeInfo()});
  ND4J_REQUIRE(p.sameShape, "execScalar: x and z must share a shape");
  if (isIntLike(x->dataType())) {
    // the scalar takes the array's type (the reference reads it as X); an INT64 scalar stays exact
    const LongType isc = s->dataType() == INT64 ? hostScalarInt64(s) : (LongType)hostScalar(s);
    prepareSpecialUse({z}, {x});
    launchIntElementwise(execStream(), k, true, x->dataType(), x->dataType(), z->dataType(), x->specialBuffer(), nullptr, z->specialBuffer(), p, isc, true);
    registerSpecialUse({z}, {x});
    return;
  }
  double sc = hostScalar(s);
  prepareSpecialUse({z}, {x});
  launchScalarOp(execStream(), k, x->dataType(), x->specialBuffer(), sc, z->specialBuffer(), p);
  registerSpecialUse({z}, {x});
  GUARD_END_VOID
}

static std::vector<LongType> hostDims(NDArray* dimension, int rank, const char* fn) {
  if (!dimension || dimension->isEmpty() || dimension->lengthOf() == 0) return {};
  ND4J_REQUIRE(dimension->buf, std::string(fn) + ": dimension array has no buffer");
  dimension->buf->syncToPrimary();
  std::vector<LongType> raw(dimension->lengthOf());
  for (LongType i = 0; i < (LongType)raw.size(); i++) {
    LongType off = 0, idx = i;
    for (int d = dimension->rankOf() - 1; d >= 0; d--) { off += (idx % dimension->sizeAt(d)) * dimension->strideAt(d); idx /= dimension->sizeAt(d); }
    if (dimension->dataType() == INT64) raw[i] = dimension->hostAs<LongType>()[off];
    else if (dimension->dataType() == INT32) raw[i] = dimension->hostAs<int>()[off];
    else ND4J_THROW(std::string(fn) + ": dimension array must be INT32 or INT64");
  }
  return normalizeDims(rank, raw.data(), (LongType)raw.size(), fn);
}

// y seen with x's shape: its non-unit dims line up with `dims` of x, its stride is 0 along every other dim
static std::vector<LongType> broadcastOperandShape(const char* fn, NDArray* x, NDArray* y, const std::vector<LongType>& dims) {
  // squeeze y's unit dims, then its remaining dims must match x along `dims`
  std::vector<LongType> yshape, ystride;
  for (int d = 0; d < y->rankOf(); d++) if (y->sizeAt(d) != 1) { yshape.push_back(y->sizeAt(d)); ystride.push_back(y->strideAt(d)); }
  std::vector<LongType> bstride(x->rankOf(), 0);
  size_t q = 0;
  for (auto d : dims) {
    if (x->sizeAt((int)d) == 1) continue;
    ND4J_REQUIRE(q < yshape.size() && yshape[q] == x->sizeAt((int)d), std::string(fn) + ": y's shape does not match x along the broadcast dimensions");
    bstride[d] = ystride[q++];
  }
  ND4J_REQUIRE(q == yshape.size(), std::string(fn) + ": y has more non-unit dims than broadcast dimensions");
  std::vector<LongType> xshape(x->rankOf());
  for (int d = 0; d < x->rankOf(); d++) xshape[d] = x->sizeAt(d);
  return makeShapeInfo(y->dataType(), 'c', xshape, bstride.data());
}
// one scalar per sub-array of x along `dims` (loops/cpu/scalar.hpp:37-80): the scalars, numbered in c order over x's other
// dims, seen with x's shape -- stride 0 along `dims`
static std::vector<LongType> scalarsPerTadShape(const char* fn, NDArray* x, NDArray* scalars, const std::vector<LongType>& dims) {
  const int rank = x->rankOf();
  std::vector<bool> inTad(rank, false);
  for (auto d : dims) inTad[d] = true;
  LongType tads = 1;
  for (int d = 0; d < rank; d++) if (!inTad[d]) tads *= x->sizeAt(d);
  ND4J_REQUIRE(scalars->lengthOf() == tads, std::string(fn) + ": " + std::to_string(scalars->lengthOf()) + " scalars for " + std::to_string(tads) + " sub-arrays");
  LongType step = 1;   // element stride of the scalars seen as a vector
  for (int d = 0; d < scalars->rankOf(); d++) if (scalars->sizeAt(d) != 1) {
    ND4J_REQUIRE(scalars->lengthOf() == scalars->sizeAt(d), std::string(fn) + ": the scalars must form a vector");
    step = scalars->strideAt(d);
  }
  std::vector<LongType> xshape(rank), st(rank, 0);
  LongType run = step;
  for (int d = rank - 1; d >= 0; d--) {
    xshape[d] = x->sizeAt(d);
    if (!inTad[d]) { st[d] = run; run *= x->sizeAt(d); }
  }
  return makeShapeInfo(scalars->dataType(), 'c', xshape, st.data());
}

// y is a smaller array whose dims line up with `dimension` of x (loops/cpu/broadcasting.hpp); realised as a
// pairwise walk in which y's stride is 0 along every other dim
void execBroadcast(Nd4jPointer* extraPointers, int opNum, OpaqueNDArray xa, OpaqueNDArray ya, OpaqueNDArray za, void*, OpaqueNDArray da) {
  OP_BEGIN(callerStream(extraPointers))
  NDArray* x = arr(xa, "execBroadcast", "x"); NDArray* y = arr(ya, "execBroadcast", "y"); NDArray* z = arr(za, "execBroadcast", "z");
  NDArray* dim = arr(da, "execBroadcast", "dimension");
  ND4J_REQUIRE(x->dataType() == z->dataType() && y->dataType() == z->dataType() && (isFloatType(z->dataType()) || isIntLike(z->dataType())),
               "execBroadcast: nd4j-hip requires X, Y and Z of one type");
  PairwiseKind k;
  switch (opNum) {  // loops/legacy_ops.h:34-39
    case 0: k = P_ADD; break; case 1: k = P_SUB; break; case 2: k = P_MUL; break; case 3: k = P_DIV; break;
    case 4: k = P_RDIV; break; case 5: k = P_RSUB; break; case 6: k = P_COPY; break;
    case 13: k = P_MIN; break; case 14: k = P_MAX; break; case 17: k = P_SQSUB; break;
    case 7: k = P_POW; break; case 15: k = P_AMIN; break; case 16: k = P_AMAX; break; case 18: k = P_FLOOR_MOD; break;
    case 19: k = P_FLOOR_DIV; break; case 20: k = P_REVERSE_MOD; break; case 21: k = P_SAFE_DIVIDE; break; case 22: k = P_MOD; break;
    case 23: k = P_TRUNCATE_DIV; break; case 26: k = P_ATAN2; break; case 27: k = P_LOGICAL_OR; break; case 28: k = P_LOGICAL_XOR; break;
    case 29: k = P_LOGICAL_NOT; break; case 30: k = P_LOGICAL_AND; break; case 31: k = P_DIVIDE_NO_NAN; break;
    case 32: k = P_IGAMMA; break; case 33: k = P_IGAMMAC; break; case 34: k = P_POW_DERIV; break;
    default: ND4J_THROW("execBroadcast: opNum " + std::to_string(opNum) + " is not implemented in nd4j-hip");
  }
  if (z->isEmpty()) return;
  auto ysi = broadcastOperandShape("execBroadcast", x, y, hostDims(dim, x->rankOf(), "execBroadcast"));
  EwPlan p = buildEwPlan({z->shapeInfo(), x->shapeInfo(), ysi.data()});
  prepareSpecialUse({z}, {x, y});
  launchPairwise(execStream(), k, x->dataType(), y->dataType(), z->dataType(), x->specialBuffer(), y->specialBuffer(), z->specialBuffer(), p);
  registerSpecialUse({z}, {x, y});
  GUARD_END_VOID
}

// ---- the bool tables: z = op(x, y) with x and y of one type and a BOOL result (loops/legacy_ops.h:30-32, 74-76, 117-119;
// loops/cpu/pairwise_bool.cpp:60-145, scalar_bool.cpp:60-140, broadcasting_bool.hpp:60-330 -- every loop calls the functor's
// three-argument form, op(x, y, extraParams)).  `ysi` describes y with x's shape (its own, or strides of 0 where it repeats).
static void boolTableImpl(const char* fn, int opNum, NDArray* x, NDArray* y, const LongType* ysi, void* extraParams, NDArray* z) {
  ND4J_REQUIRE(z->dataType() == BOOL, std::string(fn) + ": Z must be a BOOL array, got " + dtypeName(z->dataType()));
  ND4J_REQUIRE(x->dataType() == y->dataType(), std::string(fn) + ": X and Y must have one type, got " + dtypeName(x->dataType()) + ", " + dtypeName(y->dataType()));
  const DataType dt = x->dataType();
  ND4J_REQUIRE(isFloatType(dt) || dt == INT32 || dt == INT64 || dt == BOOL, std::string(fn) + ": " + dtypeName(dt) + " operands are not implemented in nd4j-hip");
  if (z->isEmpty()) return;
  EwPlan p = buildEwPlan({z->shapeInfo(), x->shapeInfo(), ysi});
  PairwiseKind k = P_EQ;
  CondKind ck = C_BOOL_AND;
  bool comparison = true;
  switch (opNum) {
    case 0: k = P_EQ; break; case 1: k = P_GT; break; case 2: k = P_LT; break; case 4: k = P_GE; break; case 6: k = P_NE; break;
    case 11: k = P_LE; break;
    case 10: k = P_NE; break;   // Not: the three-argument form is x != y (ops.h:1927-1932)
    case 3: ck = C_BOOL_EPSILON; comparison = false; break;
    case 7: ck = C_BOOL_AND; comparison = false; break; case 8: ck = C_BOOL_OR; comparison = false; break; case 9: ck = C_BOOL_XOR; comparison = false; break;
    default: ND4J_THROW(std::string(fn) + ": opNum " + std::to_string(opNum) + " is not implemented in nd4j-hip");   // 5 MatchCondition
  }
  if (comparison) {
    prepareSpecialUse({z}, {x, y});
    launchPairwise(execStream(), k, dt, dt, BOOL, x->specialBuffer(), y->specialBuffer(), z->specialBuffer(), p);
    registerSpecialUse({z}, {x, y});
    return;
  }
  CondParams c;
  c.xdt = (int)dt;
  c.mode = extraParams != nullptr ? 1 : 0;
  if (extraParams) c.compare = fetchParams(fn, extraParams, dt, 1)[0];
  // the default tolerance as the array's type holds it, static_cast<X>(1e-5): bfloat16 rounds it to 0x3728 and half to the
  // subnormal 168 * 2^-24, which are the same number; the integer types hold 0; BOOL holds true, so that every pair of
  // BOOL elements is within the tolerance (their difference, held as a BOOL, is at most true)
  c.eps = dt == DOUBLE ? 1e-5 : dt == FLOAT32 ? (double)1e-5f : isFloatType(dt) ? 168.0 / 16777216.0 : dt == BOOL ? 1.0 : 0.0;
  prepareSpecialUse({z}, {x, y});
  launchCondElementwise(execStream(), ck, c, dt, BOOL, x->specialBuffer(), y->specialBuffer(), z->specialBuffer(), p, 0.0, false);
  registerSpecialUse({z}, {x, y});
}
// y with x's shape and stride 0 everywhere: the scalar operand
static std::vector<LongType> repeatedScalarShape(NDArray* x, NDArray* s) {
  std::vector<LongType> xshape(x->rankOf()), st(x->rankOf(), 0);
  for (int d = 0; d < x->rankOf(); d++) xshape[d] = x->sizeAt(d);
  return makeShapeInfo(s->dataType(), 'c', xshape, st.data());
}
void execPairwiseTransformBool(Nd4jPointer* extraPointers, int opNum, OpaqueNDArray xa, OpaqueNDArray ya, void* extraParams, OpaqueNDArray za) {
  OP_BEGIN(callerStream(extraPointers))
  NDArray* x = arr(xa, "execPairwiseTransformBool", "x"); NDArray* y = arr(ya, "execPairwiseTransformBool", "y"); NDArray* z = arr(za, "execPairwiseTransformBool", "z");
  // a one-element y stands for a scalar (pairwise_bool.cpp:66-86); otherwise the arrays are walked by linear index
  if (y->lengthOf() == 1 && x->lengthOf() != 1) {
    auto ysi = repeatedScalarShape(x, y);
    boolTableImpl("execPairwiseTransformBool", opNum, x, y, ysi.data(), extraParams, z);
  } else {
    ND4J_REQUIRE(x->lengthOf() == y->lengthOf() && x->lengthOf() == z->lengthOf(), "execPairwiseTransformBool: x, y and z must have one length");
    boolTableImpl("execPairwiseTransformBool", opNum, x, y, y->shapeInfo(), extraParams, z);
  }
  GUARD_END_VOID
}
void execScalarBool(Nd4jPointer* extraPointers, int opNum, OpaqueNDArray xa, OpaqueNDArray za, OpaqueNDArray sa, void* extraParams) {
  OP_BEGIN(callerStream(extraPointers))
  NDArray* x = arr(xa, "execScalarBool", "x"); NDArray* z = arr(za, "execScalarBool", "z"); NDArray* s = arr(sa, "execScalarBool", "scalar");
  ND4J_REQUIRE(s->lengthOf() >= 1 && s->buf, "execScalarBool: scalar operand is empty");
  auto ysi = repeatedScalarShape(x, s);
  boolTableImpl("execScalarBool", opNum, x, s, ysi.data(), extraParams, z);
  GUARD_END_VOID
}
void execBroadcastBool(Nd4jPointer* extraPointers, int opNum, OpaqueNDArray xa, OpaqueNDArray ya, OpaqueNDArray za, void* extraParams, OpaqueNDArray da) {
  OP_BEGIN(callerStream(extraPointers))
  NDArray* x = arr(xa, "execBroadcastBool", "x"); NDArray* y = arr(ya, "execBroadcastBool", "y"); NDArray* z = arr(za, "execBroadcastBool", "z");
  NDArray* dim = arr(da, "execBroadcastBool", "dimension");
  auto ysi = broadcastOperandShape("execBroadcastBool", x, y, hostDims(dim, x->rankOf(), "execBroadcastBool"));
  boolTableImpl("execBroadcastBool", opNum, x, y, ysi.data(), extraParams, z);
  GUARD_END_VOID
}
void execScalarBoolTad(Nd4jPointer* extraPointers, int opNum, OpaqueNDArray xa, OpaqueNDArray za, OpaqueNDArray sa, void* extraParams, OpaqueNDArray da) {
  OP_BEGIN(callerStream(extraPointers))
  NDArray* x = arr(xa, "execScalarBoolTad", "x"); NDArray* z = arr(za, "execScalarBoolTad", "z"); NDArray* s = arr(sa, "execScalarBoolTad", "scalars");
  NDArray* dim = arr(da, "execScalarBoolTad", "dimension");
  auto ysi = scalarsPerTadShape("execScalarBoolTad", x, s, hostDims(dim, x->rankOf(), "execScalarBoolTad"));
  boolTableImpl("execScalarBoolTad", opNum, x, s, ysi.data(), extraParams, z);
  GUARD_END_VOID
}
// execScalar with one scalar per sub-array along `dimension` (legacy/NativeOps.h:205; loops/cpu/scalar.hpp:37-80)
void execScalarTad(Nd4jPointer* extraPointers, int opNum, OpaqueNDArray xa, OpaqueNDArray za, OpaqueNDArray sa, void*, OpaqueNDArray da) {
  OP_BEGIN(callerStream(extraPointers))
  NDArray* x = arr(xa, "execScalarTad", "x"); NDArray* z = arr(za, "execScalarTad", "z"); NDArray* s = arr(sa, "execScalarTad", "scalars");
  NDArray* dim = arr(da, "execScalarTad", "dimension");
  ND4J_REQUIRE(x->dataType() == z->dataType() && s->dataType() == z->dataType() && (isFloatType(x->dataType()) || isIntLike(x->dataType())),
               "execScalarTad: nd4j-hip requires X, the scalars and Z of one type");
  ND4J_REQUIRE(opNum != 33, "execScalarTad: CompareAndSet along a dimension is not implemented in nd4j-hip");
  const PairwiseKind k = scalarKind("execScalarTad", opNum);
  if (z->isEmpty()) return;
  auto ysi = scalarsPerTadShape("execScalarTad", x, s, hostDims(dim, x->rankOf(), "execScalarTad"));
  EwPlan p = buildEwPlan({z->shapeInfo(), x->shapeInfo(), ysi.data()});
  prepareSpecialUse({z}, {x, s});
  launchPairwise(execStream(), k, x->dataType(), s->dataType(), z->dataType(), x->specialBuffer(), s->specialBuffer(), z->specialBuffer(), p);
  registerSpecialUse({z}, {x, s});
  GUARD_END_VOID
}

}  // extern "C"
// ---- reductions of EMPTY arrays ------------------------------------------------------------------------------------
// The reference's loops give every element of Z the op's starting value when X is EMPTY (loops/cpu/reduce/reduce_same.hpp:47,
// 166-176, reduce_float.hpp:103-106,243-251, reduce_long.hpp:50-53,212-217, reduce_bool.hpp:45-48, indexreduce.hpp:106-113).
static void fillWithStart(NDArray* z, double fv, LongType iv) {
  if (z->isEmpty() || z->lengthOf() == 0) return;
  EwPlan p = buildEwPlan({z->shapeInfo(), z->shapeInfo()});
  prepareSpecialUse({z}, {});
  const DataType zdt = z->dataType();
  if (isIntLike(zdt)) launchIntElementwise(execStream(), P_COPY, true, zdt, zdt, zdt, z->specialBuffer(), nullptr, z->specialBuffer(), p, iv, true);
  else launchScalarOp(execStream(), P_COPY, zdt, z->specialBuffer(), fv, z->specialBuffer(), p);
  registerSpecialUse({z}, {});
}
// largest finite value of an integer type; DataTypeUtils::infOrMax is +inf for FLOAT and DOUBLE only and the type's largest
// value for everything else, HALF (65504) and BFLOAT16 included (array/DataTypeUtils.h:588-617)
static LongType intMax(DataType t) {
  switch (t) {
    case BOOL: return 1; case INT8: return 127; case UINT8: return 255; case INT16: return 32767; case UINT16: return 65535;
    case INT32: return 2147483647LL; case UINT32: return 4294967295LL; default: return 0x7fffffffffffffffLL;
  }
}
static void fillReduceStart(const char* fn, ReduceKind k, NDArray* x, NDArray* z) {
  const DataType xdt = x->dataType(), zdt = z->dataType();
  double fv = 0.0;
  LongType iv = 0;
  switch (k) {
    case R_PROD: fv = 1.0; iv = 1; break;                                      // ops.h:2364
    case R_MAX: case R_MIN: {                                                  // ops.h:2365-2368: -+ infOrMax<X>
      const double big = xdt == HALF ? 65504.0 : xdt == BFLOAT16 ? 3.3895313892515355e38 : (double)INFINITY;
      fv = k == R_MAX ? -big : big;
      iv = k == R_MAX ? -intMax(xdt) : intMax(xdt);
      break;
    }
    case R_AMAX: case R_AMIN:                                                  // ops.h:1225-1243: the starting value is input[0]
      ND4J_THROW(std::string(fn) + ": AMax / AMin of an EMPTY array start from the array's first element in the reference, which does not exist");
    case R_MEAN:                                                               // reduce_float.hpp:244-246: nanOrZero<Z>, NaN for FLOAT and DOUBLE only
      fv = (zdt == FLOAT32 || zdt == DOUBLE) ? (double)NAN : 0.0;
      break;
    default: break;                                                            // every other op of the two tables starts from 0
  }
  fillWithStart(z, fv, iv);
}
namespace nd4jhip {
// the ReduceFloat table when Z's type is not X's: any numeric X into any float Z (NativeOpExecutioner_reduce.cpp:34-37,104-106),
// accumulated in double by the type-agnostic kernel (the reference accumulates in float for HALF / BFLOAT16 / FLOAT results
// and in double for DOUBLE ones, ops/op_types.h:213-226)
static void runReduceFloatMixed(const char* fn, ReduceKind k, NDArray* x, NDArray* z, const std::vector<LongType>& dims) {
  runReduceMisc(fn, M_REDUCE_FLOAT, x, z, dims, false, (double)(int)k);
}
void runReduce(const char* fn, ReduceKind k, NDArray* x, NDArray* z, const std::vector<LongType>& dims) {
  const bool floatTable = k >= R_MEAN;
  if (floatTable) {
    ND4J_REQUIRE(isFloatType(z->dataType()), std::string("NativeOpExecutioner::") + fn + " requires Z operand to have floating point data type, got " + dtypeName(z->dataType()));
    ND4J_REQUIRE(isFloatType(x->dataType()) || x->dataType() == INT32 || x->dataType() == INT64 || x->dataType() == BOOL,
                 std::string(fn) + ": input type " + dtypeName(x->dataType()) + " is not implemented in nd4j-hip");
  } else {
    ND4J_REQUIRE(isFloatType(x->dataType()) || isIntLike(x->dataType()), std::string(fn) + ": this input type is not implemented in nd4j-hip");
    ND4J_REQUIRE(x->dataType() == z->dataType(), std::string("NativeOpExecutioner::") + fn + " requires both X & Z operands to have same type, got " + dtypeName(x->dataType()) + " -> " + dtypeName(z->dataType()));
  }
  if (z->isEmpty()) return;
  if (x->isEmpty()) { fillReduceStart(fn, k, x, z); return; }
  if (floatTable && x->dataType() != z->dataType()) { runReduceFloatMixed(fn, k, x, z, dims); return; }
  std::vector<LongType> d = dims;
  if (z->lengthOf() == 1 && x->lengthOf() != 1) {
    // a single output means "reduce everything" unless the kept dims are all of extent 1
    bool keptAllUnit = true;
    std::vector<bool> red(x->rankOf(), false);
    for (auto v : d) red[v] = true;
    for (int i = 0; i < x->rankOf(); i++) if (!red[i] && x->sizeAt(i) != 1) keptAllUnit = false;
    if (!keptAllUnit) d.clear();
  }
  ReducePlan p = buildReducePlan(x->shapeInfo(), z->shapeInfo(), d, false);
  auto lc = LaunchContext::defaultContext();
  prepareSpecialUse({z}, {x});
  launchReduce(lc->execStream, k, x->dataType(), z->dataType(), x->specialBuffer(), z->specialBuffer(), p, lc->reductionBuffer, LaunchContext::REDUCTION_BYTES);
  registerSpecialUse({z}, {x});
}
}  // namespace nd4jhip
extern "C" {
static ReduceKind reduceSameKind(int opNum) {
  switch (opNum) {  // loops/legacy_ops.h:100-101
    case 0: return R_SUM; case 1: return R_MAX; case 2: return R_MIN; case 3: return R_PROD; case 4: return R_ASUM;
    case 5: return R_AMAX; case 6: return R_AMIN;
    default: ND4J_THROW("execReduceSame: opNum " + std::to_string(opNum) + " is not implemented in nd4j-hip");
  }
}
static ReduceKind reduceFloatKind(int opNum) {
  switch (opNum) {  // loops/legacy_ops.h:103-105
    case 0: return R_MEAN; case 1: return R_AMEAN; case 2: return R_NORM1; case 3: return R_NORM2; case 4: return R_NORMMAX;
    case 5: return R_NORM2;  // NormFrobenius = sqrt(sum |x|^2)
    case 7: return R_SQNORM;
    case 8: return R_ENTROPY; case 9: return R_LOG_ENTROPY; case 10: return R_SHANNON_ENTROPY;
    // 6 NormP is served before this table is consulted (its exponent comes from the extra parameters)
    default: ND4J_THROW("execReduceFloat: opNum " + std::to_string(opNum) + " is not implemented in nd4j-hip");
  }
}
void execReduceSame(Nd4jPointer* extraPointers, int opNum, OpaqueNDArray xa, void*, OpaqueNDArray za) {
  OP_BEGIN(callerStream(extraPointers))
  if (xa == nullptr || za == nullptr) ND4J_THROW("execReduceSame: null pointer in input parameters");
  runReduce("execReduceSame", reduceSameKind(opNum), xa, za, {});
  GUARD_END_VOID
}
void execReduceSame2(Nd4jPointer* extraPointers, int opNum, OpaqueNDArray xa, void*, OpaqueNDArray za, OpaqueNDArray da) {
  OP_BEGIN(callerStream(extraPointers))
  if (xa == nullptr || za == nullptr || da == nullptr) ND4J_THROW("execReduceSame2: null pointer in input parameters");
  runReduce("execReduceSame2", reduceSameKind(opNum), xa, za, hostDims(da, xa->rankOf(), "execReduceSame2"));
  GUARD_END_VOID
}
// NormP (ReduceFloat 6): (sum |x|^p)^(1/p) with p = extraParams[0] in Z's type (ops.h:1280-1286)
static void runNormP(const char* fn, NDArray* x, NDArray* z, const void* extraParams, std::vector<LongType> dims) {
  ND4J_REQUIRE(isFloatType(z->dataType()), std::string("NativeOpExecutioner::") + fn + " requires Z operand to have floating point data type");
  ND4J_REQUIRE(isFloatType(x->dataType()) || x->dataType() == INT32 || x->dataType() == INT64 || x->dataType() == BOOL, std::string(fn) + ": this input type is not implemented in nd4j-hip");
  if (x->isEmpty()) { if (!z->isEmpty()) fillWithStart(z, 0.0, 0); return; }
  const double pw = fetchParams(fn, extraParams, z->dataType(), 1)[0];
  runReduceMisc(fn, M_NORMP, x, z, dims, false, pw);
}
void execReduceFloat(Nd4jPointer* extraPointers, int opNum, OpaqueNDArray xa, void* extraParams, OpaqueNDArray za) {
  OP_BEGIN(callerStream(extraPointers))
  if (xa == nullptr || za == nullptr) ND4J_THROW("execReduceFloat: null pointer in input parameters");
  if (opNum == 6) { runNormP("execReduceFloat", xa, za, extraParams, {}); return; }
  runReduce("execReduceFloat", reduceFloatKind(opNum), xa, za, {});
  GUARD_END_VOID
}
void execReduceFloat2(Nd4jPointer* extraPointers, int opNum, OpaqueNDArray xa, void* extraParams, OpaqueNDArray za, OpaqueNDArray da) {
  OP_BEGIN(callerStream(extraPointers))
  if (xa == nullptr || za == nullptr || da == nullptr) ND4J_THROW("execReduceFloat2: null pointer in input parameters");
  if (opNum == 6) { runNormP("execReduceFloat2", xa, za, extraParams, hostDims(da, xa->rankOf(), "execReduceFloat2")); return; }
  runReduce("execReduceFloat2", reduceFloatKind(opNum), xa, za, hostDims(da, xa->rankOf(), "execReduceFloat2"));
  GUARD_END_VOID
}

// reductions with their own accumulator / output types
}  // extern "C"
namespace nd4jhip {
void runReduceMisc(const char* fn, MiscReduceKind k, NDArray* x, NDArray* z, std::vector<LongType> d, bool biasCorrected, double param) {
  if (z->isEmpty()) return;
  if (x->isEmpty()) {
    // the starting values of the counting, Any / All and NormP ops (ops.h:1180-1215,1139-1163,1280-1286); the summary
    // statistics initialise from x[0], which an EMPTY array does not have (loops/cpu/summarystatsreduce.cpp:106-113)
    ND4J_REQUIRE(k != M_VARIANCE && k != M_STDDEV, std::string(fn) + ": the reference initialises the statistics of an EMPTY array from its first element, which does not exist");
    fillWithStart(z, k == M_ALL ? 1.0 : 0.0, k == M_ALL ? 1 : 0);
    return;
  }
  if (z->lengthOf() == 1 && x->lengthOf() != 1) {
    bool keptAllUnit = true;
    std::vector<bool> red(x->rankOf(), false);
    for (auto v : d) red[v] = true;
    for (int i = 0; i < x->rankOf(); i++) if (!red[i] && x->sizeAt(i) != 1) keptAllUnit = false;
    if (!keptAllUnit) d.clear();
  }
  ReducePlan p = buildReducePlan(x->shapeInfo(), z->shapeInfo(), d, false);
  auto lc = LaunchContext::defaultContext();
  prepareSpecialUse({z}, {x});
  launchReduceMisc(lc->execStream, k, x->dataType(), z->dataType(), x->specialBuffer(), z->specialBuffer(), p, biasCorrected,
                   lc->reductionBuffer, LaunchContext::REDUCTION_BYTES, nullptr, FLOAT32, nullptr, param);
  registerSpecialUse({z}, {x});
}
}  // namespace nd4jhip
extern "C" {
// reduce3: z[o] = f(x tad o, y tad o) with y shaped like x (loops/cpu/reduce3.hpp); opNums loops/legacy_ops.h:88-90
static void runReduce3(const char* fn, int opNum, NDArray* x, NDArray* y, NDArray* z, std::vector<LongType> d, const void* extraParams = nullptr) {
  MiscReduceKind k;
  double param = 0.0;
  switch (opNum) {
    case 0: k = M3_MANHATTAN; break; case 1: k = M3_EUCLIDEAN; break; case 2: k = M3_COSINE_SIMILARITY; break; case 3: k = M3_DOT; break;
    case 5: k = M3_COSINE_DISTANCE; break; case 6: k = M3_JACCARD; break; case 7: k = M3_HAMMING; break;
    case 4: k = M3_EQUALS_EPS; break;   // the tolerance is the third extra parameter, in Z's type (op_macros_special.h:449-457)
    default: ND4J_THROW(std::string(fn) + ": opNum " + std::to_string(opNum) + " is not implemented in nd4j-hip");
  }
  if (opNum == 4 && isFloatType(z->dataType())) param = fetchParams(fn, extraParams, z->dataType(), 3)[2];
  ND4J_REQUIRE(isFloatType(z->dataType()), std::string(fn) + ": Z must have a floating point type");
  ND4J_REQUIRE(x->rankOf() == y->rankOf() && x->lengthOf() == y->lengthOf(), std::string(fn) + ": x and y must have the same shape");
  for (int i = 0; i < x->rankOf(); i++) ND4J_REQUIRE(x->sizeAt(i) == y->sizeAt(i), std::string(fn) + ": x and y must have the same shape");
  // an EMPTY operand: the reference's loop over x's (zero) elements writes nothing (loops/cpu/reduce3.hpp:49-57)
  if (z->isEmpty() || x->isEmpty() || y->isEmpty()) return;
  if (z->lengthOf() == 1 && x->lengthOf() != 1) {
    bool keptAllUnit = true;
    std::vector<bool> red(x->rankOf(), false);
    for (auto v : d) red[v] = true;
    for (int i = 0; i < x->rankOf(); i++) if (!red[i] && x->sizeAt(i) != 1) keptAllUnit = false;
    if (!keptAllUnit) d.clear();
  }
  ReducePlan p = buildReducePlan(x->shapeInfo(), z->shapeInfo(), d, false);
  ReducePlan py = buildReducePlan(y->shapeInfo(), z->shapeInfo(), d, false);
  auto lc = LaunchContext::defaultContext();
  prepareSpecialUse({z}, {x, y});
  launchReduceMisc(lc->execStream, k, x->dataType(), z->dataType(), x->specialBuffer(), z->specialBuffer(), p, false, lc->reductionBuffer,
                   LaunchContext::REDUCTION_BYTES, y->specialBuffer(), y->dataType(), &py, param);
  registerSpecialUse({z}, {x, y});
}
static MiscReduceKind summaryKind(int opNum) {
  switch (opNum) {  // loops/legacy_ops.h:69
    case 0: return M_VARIANCE; case 1: return M_STDDEV;
    default: ND4J_THROW("execSummaryStats: opNum " + std::to_string(opNum) + " is not implemented in nd4j-hip");
  }
}
extern "C" {
void execSummaryStatsScalar(Nd4jPointer* extraPointers, int opNum, OpaqueNDArray xa, void*, OpaqueNDArray za, bool biasCorrected) {
  OP_BEGIN(callerStream(extraPointers))
  NDArray* x = arr(xa, "execSummaryStatsScalar", "x"); NDArray* z = arr(za, "execSummaryStatsScalar", "z");
  ND4J_REQUIRE(isFloatType(z->dataType()), "execSummaryStatsScalar: Z must have a floating point type");
  runReduceMisc("execSummaryStatsScalar", summaryKind(opNum), x, z, {}, biasCorrected);
  GUARD_END_VOID
}
void execSummaryStatsTad(Nd4jPointer* extraPointers, int opNum, OpaqueNDArray xa, void*, OpaqueNDArray za, OpaqueNDArray da, bool biasCorrected) {
  OP_BEGIN(callerStream(extraPointers))
  NDArray* x = arr(xa, "execSummaryStatsTad", "x"); NDArray* z = arr(za, "execSummaryStatsTad", "z");
  ND4J_REQUIRE(isFloatType(z->dataType()), "execSummaryStatsTad: Z must have a floating point type");
  runReduceMisc("execSummaryStatsTad", summaryKind(opNum), x, z, hostDims(da, x->rankOf(), "execSummaryStatsTad"), biasCorrected);
  GUARD_END_VOID
}
}  // extern "C"
// MatchCondition (count), FirstIndex / LastIndex: [compare, eps, mode] in X's type
static void runCondReduce(const char* fn, CondReduceKind kind, NDArray* x, NDArray* z, std::vector<LongType> d, const void* extraParams) {
  ND4J_REQUIRE(isFloatType(x->dataType()) || x->dataType() == INT32 || x->dataType() == INT64, std::string(fn) + ": match conditions take float, INT32 or INT64 arrays here");
  if (z->isEmpty()) return;
  // EMPTY x: a count of 0 (reduce_long.hpp:50-53,212-217), no index (-1, ops.h:2079-2085,2123-2129)
  if (x->isEmpty()) { fillWithStart(z, kind == CR_COUNT ? 0.0 : -1.0, kind == CR_COUNT ? 0 : -1); return; }
  const CondParams c = condParams(fn, extraParams, x->dataType(), false);
  if (z->lengthOf() == 1 && x->lengthOf() != 1) {
    bool keptAllUnit = true;
    std::vector<bool> red(x->rankOf(), false);
    for (auto v : d) red[v] = true;
    for (int i = 0; i < x->rankOf(); i++) if (!red[i] && x->sizeAt(i) != 1) keptAllUnit = false;
    if (!keptAllUnit) d.clear();
  }
  ReducePlan p = buildReducePlan(x->shapeInfo(), z->shapeInfo(), d, false);
  auto lc = LaunchContext::defaultContext();
  prepareSpecialUse({z}, {x});
  launchCondReduce(lc->execStream, kind, c, z->dataType(), x->specialBuffer(), z->specialBuffer(), p, lc->reductionBuffer, LaunchContext::REDUCTION_BYTES);
  registerSpecialUse({z}, {x});
}
extern "C" {
static void reduceLong(const char* fn, int opNum, OpaqueNDArray xa, OpaqueNDArray za, OpaqueNDArray da, const void* extraParams) {
  NDArray* x = arr(xa, fn, "x"); NDArray* z = arr(za, fn, "z");
  ND4J_REQUIRE(z->dataType() == INT64, std::string("NativeOpExecutioner::execReduceLong wrong Z data type: Z must be INT64, got ") + dtypeName(z->dataType()));
  if (opNum == 2) {   // MatchCondition (loops/legacy_ops.h:95)
    runCondReduce(fn, CR_COUNT, x, z, da ? hostDims(da, x->rankOf(), fn) : std::vector<LongType>{}, extraParams);
    return;
  }
  MiscReduceKind k;
  switch (opNum) {  // loops/legacy_ops.h:95
    case 0: k = M_COUNT_NONZERO; break; case 1: k = M_COUNT_ZERO; break;
    default: ND4J_THROW(std::string(fn) + ": opNum " + std::to_string(opNum) + " is not implemented in nd4j-hip");
  }
  runReduceMisc(fn, k, x, z, da ? hostDims(da, x->rankOf(), fn) : std::vector<LongType>{}, false);
}
void execReduceLong(Nd4jPointer* extraPointers, int opNum, OpaqueNDArray xa, void* extraParams, OpaqueNDArray za, OpaqueNDArray da) {
  OP_BEGIN(callerStream(extraPointers))
  reduceLong("execReduceLong", opNum, xa, za, da, extraParams);
  GUARD_END_VOID
}
void execReduceLong2(Nd4jPointer* extraPointers, int opNum, OpaqueNDArray xa, void* extraParams, OpaqueNDArray za, OpaqueNDArray da) {
  OP_BEGIN(callerStream(extraPointers))
  reduceLong("execReduceLong2", opNum, xa, za, da, extraParams);
  GUARD_END_VOID
}
static void reduceBool(const char* fn, int opNum, OpaqueNDArray xa, OpaqueNDArray za, OpaqueNDArray da) {
  NDArray* x = arr(xa, fn, "x"); NDArray* z = arr(za, fn, "z");
  ND4J_REQUIRE(z->dataType() == BOOL, std::string("NativeOpExecutioner::execReduceBool requires Z operand to have BOOL type, got ") + dtypeName(z->dataType()));
  MiscReduceKind k;
  switch (opNum) {  // loops/legacy_ops.h:97-98
    case 0: k = M_ANY; break; case 1: k = M_ALL; break; case 2: k = M_ANY_FINITE; break; case 3: k = M_ANY_INF_OR_NAN; break;
    case 4: k = M_ANY_NAN; break; case 5: k = M_ANY_INF; break; case 6: k = M_ANY_POSITIVE; break; case 7: k = M_ANY_NEGATIVE; break;
    default: ND4J_THROW(std::string(fn) + ": opNum " + std::to_string(opNum) + " is not implemented in nd4j-hip");
  }
  runReduceMisc(fn, k, x, z, da ? hostDims(da, x->rankOf(), fn) : std::vector<LongType>{}, false);
}
void execReduceBool(Nd4jPointer* extraPointers, int opNum, OpaqueNDArray xa, void*, OpaqueNDArray za, OpaqueNDArray da) {
  OP_BEGIN(callerStream(extraPointers))
  reduceBool("execReduceBool", opNum, xa, za, da);
  GUARD_END_VOID
}
void execReduceBool2(Nd4jPointer* extraPointers, int opNum, OpaqueNDArray xa, void*, OpaqueNDArray za, OpaqueNDArray da) {
  OP_BEGIN(callerStream(extraPointers))
  reduceBool("execReduceBool2", opNum, xa, za, da);
  GUARD_END_VOID
}
void execReduce3(Nd4jPointer* extraPointers, int opNum, OpaqueNDArray xa, void* extraParams, OpaqueNDArray ya, OpaqueNDArray za) {
  OP_BEGIN(callerStream(extraPointers))
  runReduce3("execReduce3", opNum, arr(xa, "execReduce3", "x"), arr(ya, "execReduce3", "y"), arr(za, "execReduce3", "z"), {}, extraParams);
  GUARD_END_VOID
}
void execReduce3Scalar(Nd4jPointer* extraPointers, int opNum, OpaqueNDArray xa, void* extraParams, OpaqueNDArray ya, OpaqueNDArray za) {
  OP_BEGIN(callerStream(extraPointers))
  runReduce3("execReduce3Scalar", opNum, arr(xa, "execReduce3Scalar", "x"), arr(ya, "execReduce3Scalar", "y"), arr(za, "execReduce3Scalar", "z"), {}, extraParams);
  GUARD_END_VOID
}
void execReduce3Tad(Nd4jPointer* extraPointers, int opNum, OpaqueNDArray xa, void* extraParams, OpaqueNDArray ya, OpaqueNDArray za, OpaqueNDArray da) {
  OP_BEGIN(callerStream(extraPointers))
  NDArray* x = arr(xa, "execReduce3Tad", "x");
  runReduce3("execReduce3Tad", opNum, x, arr(ya, "execReduce3Tad", "y"), arr(za, "execReduce3Tad", "z"), hostDims(da, x->rankOf(), "execReduce3Tad"), extraParams);
  GUARD_END_VOID
}
// every sub-array of x along `dimension` against every sub-array of y along it: z[i][j] = f(x tad i, y tad j), the
// sub-arrays numbered in c order over the other dims (loops/cpu/reduce3.hpp execAll).  Realised as execReduce3Tad on two
// views of rank |x's other dims| + |y's other dims| + |dimension|, x repeated (stride 0) along y's dims and y along x's.
void execReduce3All(Nd4jPointer* extraPointers, int opNum, OpaqueNDArray xa, OpaqueNDArray ya, OpaqueNDArray za, OpaqueNDArray da, void* extraParams) {
  OP_BEGIN(callerStream(extraPointers))
  const char* fn = "execReduce3All";
  NDArray* x = arr(xa, fn, "x"); NDArray* y = arr(ya, fn, "y"); NDArray* z = arr(za, fn, "z");
  ND4J_REQUIRE(x->rankOf() == y->rankOf(), std::string(fn) + ": x and y must have one rank");
  if (x->isEmpty() || y->isEmpty()) return;   // nothing is written (loops/cpu/reduce3.hpp:49-57)
  const int rank = x->rankOf();
  auto dims = hostDims(da, rank, fn);
  ND4J_REQUIRE(!dims.empty(), std::string(fn) + ": the dimensions of the sub-arrays are required");
  std::vector<bool> inTad(rank, false);
  for (auto d : dims) { inTad[d] = true; ND4J_REQUIRE(x->sizeAt((int)d) == y->sizeAt((int)d), std::string(fn) + ": the sub-arrays of x and y must have one shape"); }
  std::vector<LongType> shape, xs, ys, zs;
  LongType nx = 1, ny = 1;
  for (int d = 0; d < rank; d++) if (!inTad[d]) { nx *= x->sizeAt(d); ny *= y->sizeAt(d); }
  ND4J_REQUIRE(z->lengthOf() == nx * ny, std::string(fn) + ": z must hold " + std::to_string(nx) + " x " + std::to_string(ny) + " results");
  if (z->isEmpty()) return;
  // z as [nx, ny]: its own two dims when it has that shape, else a dense c-order array
  LongType zRow = ny, zCol = 1;
  if (z->rankOf() == 2 && z->sizeAt(0) == nx && z->sizeAt(1) == ny) { zRow = z->strideAt(0); zCol = z->strideAt(1); }
  else {
    bool dense = true;
    LongType expect = 1;
    for (int d = z->rankOf() - 1; d >= 0; d--) { if (z->sizeAt(d) != 1 && z->strideAt(d) != expect) dense = false; expect *= z->sizeAt(d); }
    ND4J_REQUIRE(dense, std::string(fn) + ": z must have shape [sub-arrays of x, sub-arrays of y] or be dense in c order");
  }
  LongType run = zRow * nx;
  for (int d = 0; d < rank; d++) if (!inTad[d]) { run /= x->sizeAt(d); shape.push_back(x->sizeAt(d)); xs.push_back(x->strideAt(d)); ys.push_back(0); zs.push_back(run); }
  run = zCol * ny;
  for (int d = 0; d < rank; d++) if (!inTad[d]) { run /= y->sizeAt(d); shape.push_back(y->sizeAt(d)); xs.push_back(0); ys.push_back(y->strideAt(d)); zs.push_back(run); }
  std::vector<LongType> tadAxes;
  const size_t outRank = shape.size();
  std::vector<LongType> zshape(shape.begin(), shape.end());
  for (auto d : dims) { tadAxes.push_back((LongType)shape.size()); shape.push_back(x->sizeAt((int)d)); xs.push_back(x->strideAt((int)d)); ys.push_back(y->strideAt((int)d)); }
  ND4J_REQUIRE((int)shape.size() <= MAX_RANK, std::string(fn) + ": too many dims");
  NDArray xv = *x, yv = *y, zv = *z;
  xv.si = makeShapeInfo(x->dataType(), 'c', shape, xs.data());
  yv.si = makeShapeInfo(y->dataType(), 'c', shape, ys.data());
  if (outRank == 0) { zshape = {1}; zs = {1}; }
  zv.si = makeShapeInfo(z->dataType(), 'c', zshape, zs.data());
  runReduce3(fn, opNum, &xv, &yv, &zv, tadAxes, extraParams);
  GUARD_END_VOID
}
void execTransformBool(Nd4jPointer* extraPointers, int opNum, OpaqueNDArray xa, void* extraParams, OpaqueNDArray za) {
  OP_BEGIN(callerStream(extraPointers))
  NDArray* x = arr(xa, "execTransformBool", "x"); NDArray* z = arr(za, "execTransformBool", "z");
  ND4J_REQUIRE(z->dataType() == BOOL, std::string("NativeOpExecutioner::execTransformBool requires Z to have same boolean type, got ") + dtypeName(z->dataType()));
  ND4J_REQUIRE(isFloatType(x->dataType()) || isIntLike(x->dataType()), "execTransformBool: this input type is not implemented in nd4j-hip");
  if (opNum == 5) {   // MatchConditionBool (loops/legacy_ops.h:50)
    ND4J_REQUIRE(isFloatType(x->dataType()) || x->dataType() == INT32 || x->dataType() == INT64, "execTransformBool: MatchConditionBool takes float, INT32 or INT64 arrays here");
    if (x->isEmpty() || z->isEmpty()) return;
    const CondParams c = condParams("execTransformBool", extraParams, x->dataType(), false);
    EwPlan p = buildEwPlan({z->shapeInfo(), x->shapeInfo()});
    prepareSpecialUse({z}, {x});
    launchCondElementwise(execStream(), C_MATCH_BOOL, c, x->dataType(), BOOL, x->specialBuffer(), nullptr, z->specialBuffer(), p, 0.0, false);
    registerSpecialUse({z}, {x});
    return;
  }
  UnaryKind k;
  switch (opNum) {  // loops/legacy_ops.h:49-51
    case 1: k = U_IS_INF; break; case 2: k = U_IS_NAN; break; case 3: k = U_IS_FINITE; break; case 4: k = U_IS_INF_OR_NAN; break;
    case 6: k = U_IS_POSITIVE; break; case 7: k = U_NOT; break; case 8: k = U_IS_NEGATIVE; break;
    default: ND4J_THROW("execTransformBool: opNum " + std::to_string(opNum) + " is not implemented in nd4j-hip");
  }
  runUnary("execTransformBool", k, x, z);
  GUARD_END_VOID
}
}  // extern "C"

static IndexKind indexKind(int opNum) {
  switch (opNum) {  // loops/legacy_ops.h:131-132
    case 0: return I_MAX; case 1: return I_MIN; case 2: return I_AMAX; case 3: return I_AMIN;
    default: ND4J_THROW("execIndexReduce: opNum " + std::to_string(opNum) + " is not implemented in nd4j-hip");
  }
}
}  // extern "C"
namespace nd4jhip {
void runIndexReduce(const char* fn, int opNum, NDArray* x, NDArray* z, const std::vector<LongType>& dims) {
  ND4J_REQUIRE(isFloatType(x->dataType()) || isIntLike(x->dataType()), std::string(fn) + ": this input type is not implemented in nd4j-hip");
  ND4J_REQUIRE(z->dataType() == INT64 || z->dataType() == INT32,
               std::string("NativeOpExecutioner::") + fn + " requires Z operand to have INT32/INT64 type, got " + dtypeName(z->dataType()));
  if (z->isEmpty()) return;
  IndexKind k = indexKind(opNum);
  // EMPTY x: the starting pair's index, 0 (loops/cpu/indexreduce.hpp:106-113, ops/op_macros_index_reduce.h:46-51)
  if (x->isEmpty()) { fillWithStart(z, 0.0, 0); return; }
  std::vector<LongType> d = dims;
  if (z->lengthOf() == 1 && (int)d.size() < x->rankOf()) {
    bool keptAllUnit = true;
    std::vector<bool> red(x->rankOf(), false);
    for (auto v : d) red[v] = true;
    for (int i = 0; i < x->rankOf(); i++) if (!red[i] && x->sizeAt(i) != 1) keptAllUnit = false;
    if (!keptAllUnit) d.clear();
  }
  // z is addressed linearly, z[i] for the i-th sub-array (helpers/cpu/loops/IndexReductionLoops.hpp:61-75);
  // with a dense z that is also what walking its shape gives
  ReducePlan p = buildReducePlan(x->shapeInfo(), z->shapeInfo(), d, false);
  auto lc = LaunchContext::defaultContext();
  prepareSpecialUse({z}, {x});
  launchIndexReduce(lc->execStream, k, x->dataType(), z->dataType(), x->specialBuffer(), z->specialBuffer(), p, lc->reductionBuffer, LaunchContext::REDUCTION_BYTES);
  registerSpecialUse({z}, {x});
}
}  // namespace nd4jhip
extern "C" {
void execIndexReduce(Nd4jPointer* extraPointers, int opNum, OpaqueNDArray xa, void* extraParams, OpaqueNDArray za, OpaqueNDArray da) {
  OP_BEGIN(callerStream(extraPointers))
  NDArray* x = arr(xa, "execIndexReduce", "x"); NDArray* z = arr(za, "execIndexReduce", "z"); NDArray* d = arr(da, "execIndexReduce", "dimension");
  if (opNum == 4 || opNum == 5) {   // FirstIndex, LastIndex (loops/legacy_ops.h:132): -1 where nothing matches
    ND4J_REQUIRE(z->dataType() == INT64 || z->dataType() == INT32, "NativeOpExecutioner::execIndexReduce requires Z operand to have INT32/INT64 type");
    runCondReduce("execIndexReduce", opNum == 4 ? CR_FIRST : CR_LAST, x, z, hostDims(d, x->rankOf(), "execIndexReduce"), extraParams);
    return;
  }
  runIndexReduce("execIndexReduce", opNum, x, z, hostDims(d, x->rankOf(), "execIndexReduce"));
  GUARD_END_VOID
}
void execIndexReduceScalar(Nd4jPointer* extraPointers, int opNum, OpaqueNDArray xa, void* extraParams, OpaqueNDArray za) {
  OP_BEGIN(callerStream(extraPointers))
  NDArray* x = arr(xa, "execIndexReduceScalar", "x"); NDArray* z = arr(za, "execIndexReduceScalar", "z");
  if (opNum == 4 || opNum == 5) {
    ND4J_REQUIRE(z->dataType() == INT64 || z->dataType() == INT32, "NativeOpExecutioner::execIndexReduceScalar requires Z operand to have INT32/INT64 type");
    runCondReduce("execIndexReduceScalar", opNum == 4 ? CR_FIRST : CR_LAST, x, z, {}, extraParams);
    return;
  }
  runIndexReduce("execIndexReduceScalar", opNum, x, z, {});
  GUARD_END_VOID
}

// ---- op context ---------------------------------------------------------------------------------------------
OpaqueContext* createGraphContext(int nodeId) {
  auto* c = new Nd4jHipContext();
  c->nodeId = nodeId;
  return c;
}
void deleteGraphContext(OpaqueContext* ptr) { delete ptr; }
void setGraphContextCudaContext(OpaqueContext* ptr, void* stream, void* reductionPointer, void* allocationPointer) {
  if (!ptr) return;
  ptr->callerStream = stream; ptr->callerReduction = reductionPointer; ptr->callerAllocation = allocationPointer;
}
void markGraphContextInplace(OpaqueContext* ptr, bool v) { if (ptr) ptr->inplace = v; }
static void setAt(std::vector<NDArray*>& v, int index, NDArray* a) {
  if (index < 0) ND4J_THROW("graph context: negative array index");
  if ((int)v.size() <= index) v.resize(index + 1, nullptr);
  v[index] = a;
}
void setGraphContextInputArray(OpaqueContext* ptr, int index, OpaqueNDArray a) {
  GUARD_BEGIN
  if (a == nullptr) ND4J_THROW("setGraphContextInputArray: Input arrays were null!");
  ND4J_REQUIRE(ptr != nullptr, "setGraphContextInputArray: Context was null!");
  setAt(ptr->inputs, index, a);
  GUARD_END_VOID
}
void setGraphContextOutputArray(OpaqueContext* ptr, int index, OpaqueNDArray a) {
  GUARD_BEGIN
  if (a == nullptr) ND4J_THROW("setGraphContextOutputArray: Input arrays were null!");
  ND4J_REQUIRE(ptr != nullptr, "setGraphContextOutputArray: Context was null!");
  setAt(ptr->outputs, index, a);
  GUARD_END_VOID
}
void setGraphContextInputArraysArr(OpaqueContext* ptr, int n, OpaqueNDArrayArr a) {
  GUARD_BEGIN
  if (a == nullptr) ND4J_THROW("setGraphContextInputArraysArr: Input arrays were null!");
  if (ptr == nullptr) ND4J_THROW("setGraphContextInputArraysArr: Context was null!");
  for (int i = 0; i < n; i++) {
    if (a[i] == nullptr) ND4J_THROW("setGraphContextInputArraysArr: Input array at index " + std::to_string(i) + " was null!");
    setAt(ptr->inputs, i, a[i]);
  }
  GUARD_END_VOID
}
void setGraphContextOutputArraysArr(OpaqueContext* ptr, int n, OpaqueNDArrayArr a) {
  GUARD_BEGIN
  if (a == nullptr) ND4J_THROW("setGraphContextOutputArraysArr: Output arrays were null!");
  if (ptr == nullptr) ND4J_THROW("setGraphContextOutputArraysArr: Context was null!");
  for (int i = 0; i < n; i++) {
    if (a[i] == nullptr) ND4J_THROW("setGraphContextOutputArraysArr: Output array at index " + std::to_string(i) + " was null!");
    setAt(ptr->outputs, i, a[i]);
  }
  GUARD_END_VOID
}
void setGraphContextTArguments(OpaqueContext* ptr, double* a, int n) { if (ptr) ptr->tArgs.assign(a, a + (n > 0 ? n : 0)); }
void setGraphContextIArguments(OpaqueContext* ptr, Nd4jLong* a, int n) { if (ptr) ptr->iArgs.assign(a, a + (n > 0 ? n : 0)); }
void setGraphContextBArguments(OpaqueContext* ptr, bool* a, int n) { if (ptr) ptr->bArgs.assign(a, a + (n > 0 ? n : 0)); }
void setGraphContextDArguments(OpaqueContext* ptr, int* a, int n) {
  if (!ptr) return;
  ptr->dArgs.clear();
  for (int i = 0; i < n; i++) ptr->dArgs.push_back((DataType)a[i]);
}
void ctxAllowHelpers(OpaqueContext* ptr, bool v) { if (ptr) ptr->helpersAllowed = v; }
void ctxShapeFunctionOverride(OpaqueContext* ptr, bool v) { if (ptr) ptr->shapeFunctionOverride = v; }
void ctxSetExecutionMode(OpaqueContext* ptr, int m) { if (ptr) ptr->execMode = m; }
void ctxPurge(OpaqueContext* ptr) {
  if (!ptr) return;
  ptr->inputs.clear(); ptr->outputs.clear(); ptr->tArgs.clear(); ptr->iArgs.clear(); ptr->bArgs.clear(); ptr->dArgs.clear();
}
OpaqueNDArray getInputArrayNative(OpaqueContext* ptr, int idx) {
  if (!ptr || idx < 0 || idx >= (int)ptr->inputs.size()) return nullptr;
  return static_cast<OpaqueNDArray>(ptr->inputs[idx]);
}
OpaqueNDArray getOutputArrayNative(OpaqueContext* ptr, int idx) {
  if (!ptr || idx < 0 || idx >= (int)ptr->outputs.size()) return nullptr;
  return static_cast<OpaqueNDArray>(ptr->outputs[idx]);
}
Nd4jLong numInputsNative(OpaqueContext* ptr) { return ptr ? (Nd4jLong)ptr->inputs.size() : 0; }
Nd4jLong numOutputsNative(OpaqueContext* ptr) { return ptr ? (Nd4jLong)ptr->outputs.size() : 0; }
Nd4jLong numTArgumentsNative(OpaqueContext* ptr) { return ptr ? (Nd4jLong)ptr->tArgs.size() : 0; }
Nd4jLong numIArgumentsNative(OpaqueContext* ptr) { return ptr ? (Nd4jLong)ptr->iArgs.size() : 0; }
Nd4jLong numBNative(OpaqueContext* ptr) { return ptr ? (Nd4jLong)ptr->bArgs.size() : 0; }
Nd4jLong numDNative(OpaqueContext* ptr) { return ptr ? (Nd4jLong)ptr->dArgs.size() : 0; }
double tArgumentNative(OpaqueContext* ptr, int idx) { return ptr && idx >= 0 && idx < (int)ptr->tArgs.size() ? ptr->tArgs[idx] : 0.0; }
Nd4jLong iArgumentAtNative(OpaqueContext* ptr, int idx) { return ptr && idx >= 0 && idx < (int)ptr->iArgs.size() ? ptr->iArgs[idx] : 0; }
bool bArgAtNative(OpaqueContext* ptr, int idx) { return ptr && idx >= 0 && idx < (int)ptr->bArgs.size() ? (bool)ptr->bArgs[idx] : false; }
Nd4jLong dataTypeNativeAt(OpaqueContext* ptr, int idx) { return ptr && idx >= 0 && idx < (int)ptr->dArgs.size() ? (Nd4jLong)ptr->dArgs[idx] : 0; }

// ---- declarable ops --------------------------------------------------------------------------------------------
const char* getAllCustomOps(void) { return ops::allCustomOps(); }
Nd4jLong nd4jhipOpHash(const char* name) { return name ? ops::opHash(name) : 0; }

Nd4jStatus execCustomOp2(Nd4jPointer* extraPointers, Nd4jLong hash, OpaqueContext* ctx) {
  OP_BEGIN(ctx && ctx->callerStream ? ctx->callerStream : callerStream(extraPointers))
  ND4J_REQUIRE(ctx != nullptr, "execCustomOp2: context is null");
  const ops::OpDescriptor* op = ops::findOp(hash);
  if (!op) ND4J_THROW("execCustomOp2: unknown op hash " + std::to_string(hash) + " (op is not implemented in nd4j-hip)");
  ops::executeOp(*op, *ctx);
  if (captureActive()) {
    RecordedOp rec;   // run stays empty: a custom op is replayed from this record's own copy of the context
    rec.kind = RecordedOp::CUSTOM; rec.op = op; rec.ctx = *ctx;
    recordOp(std::move(rec));
  }
  if (Environment::get().syncAfterCustomOp) HIP_CHECK(hipStreamSynchronize(execStream()));
  return 0;
  GUARD_END(1)
}
OpaqueShapeList* calculateOutputShapes2(Nd4jPointer*, Nd4jLong hash, OpaqueContext* ctx) {
  GUARD_BEGIN
  ND4J_REQUIRE(ctx != nullptr, "calculateOutputShapes2: context is null");
  const ops::OpDescriptor* op = ops::findOp(hash);
  if (!op) ND4J_THROW("calculateOutputShapes2: unknown op hash " + std::to_string(hash));
  auto* list = new Nd4jHipShapeList();
  try {
    for (auto& si : op->shapeFn(*ctx)) list->shapes.push_back(cachedShapeBuffer(si.data()));
  } catch (...) { delete list; throw; }
  return list;
  GUARD_END(nullptr)
}
Nd4jLong getShapeListSize(OpaqueShapeList* list) { return list ? (Nd4jLong)list->shapes.size() : 0; }
const Nd4jLong* getShape(OpaqueShapeList* list, Nd4jLong i) {
  if (!list || i < 0 || i >= (Nd4jLong)list->shapes.size()) return nullptr;
  return list->shapes[i]->primary();
}
void deleteShapeList(Nd4jPointer shapeList) { delete static_cast<Nd4jHipShapeList*>(shapeList); }

void nd4jhipSetSyncAfterCustomOp(int enable) { Environment::get().syncAfterCustomOp = enable != 0; }

// ---- stream capture: a launch-bound sequence of ops recorded once and replayed as one HIP graph -----------------------
namespace {
struct CapturedGraph {
  hipGraph_t graph = nullptr;
  hipGraphExec_t exec = nullptr;
  CaptureRecord record;           // the buffers the recorded kernels read and write
  std::vector<RecordedOp> ops;    // the op calls the facade recognised, in call order
  int opCalls = 0;                // every op entry point called during the capture
  int fusedOps = 0;               // ops that the merged plan gives to a neighbour's kernel
  int fusedApplied = 0;           // ... and how many of them ran there the last time the plan was executed
  std::vector<std::function<void()>> plan;   // the merged sequence as ordinary launches (empty: a call went unrecorded)
};
// how nd4jhipGraphLaunch replays: 0 the instantiated HIP graph, 1 the merged sequence launched kernel by kernel
int g_graphReplayMode = [] { const char* v = getenv("ND4JHIP_GRAPH_REPLAY"); return v != nullptr && std::string(v) == "kernels" ? 1 : 0; }();
CapturedGraph* g_openCapture = nullptr;
bool g_syncBeforeCapture = true;
bool graphFusionEnabled() {
  static const bool on = [] { const char* v = getenv("ND4JHIP_GRAPH_FUSION"); return v == nullptr || atoi(v) != 0; }();
  return on;
}
}
}  // extern "C"
static void recordOp(RecordedOp&& r) {
  if (!g_openCapture) return;
  r.adopt();   // the record keeps its own views of the arrays from here on: the caller may delete its handles before End
  g_openCapture->ops.push_back(std::move(r));
}
extern "C" {
int nd4jhipGraphBeginCapture(void) {
  GRAPH_BEGIN
  ND4J_REQUIRE(!captureActive(), "nd4jhipGraphBeginCapture: a capture is already in progress");
  // every op call between begin and end records its kernels instead of running them: nothing may wait on the stream
  g_syncBeforeCapture = Environment::get().syncAfterCustomOp;
  Environment::get().syncAfterCustomOp = false;
  HIP_CHECK(hipStreamSynchronize(execStream()));
  HIP_CHECK(hipStreamBeginCapture(execStream(), hipStreamCaptureModeRelaxed));
  g_openCapture = new CapturedGraph();
  g_captureOpCalls = &g_openCapture->opCalls;
  setActiveCapture(&g_openCapture->record);
  return 0;
  GUARD_END(1)
}
Nd4jPointer nd4jhipGraphEndCapture(void) {
  GRAPH_BEGIN
  ND4J_REQUIRE(captureActive() && g_openCapture, "nd4jhipGraphEndCapture: no capture in progress");
  // Whatever happens below, the capture is closed and, unless the graph is handed to the caller, freed.
  struct Closer {
    CapturedGraph* cg;
    bool streamOpen = true;    // the stream is still in capture mode
    ~Closer() {
      if (streamOpen) { hipGraph_t dropped = nullptr; (void)hipStreamEndCapture(execStream(), &dropped); if (dropped) (void)hipGraphDestroy(dropped); (void)hipGetLastError(); }
      g_openCapture = nullptr;
      g_captureOpCalls = nullptr;
      setActiveCapture(nullptr);
      Environment::get().syncAfterCustomOp = g_syncBeforeCapture;
      if (cg) { if (cg->exec) (void)hipGraphExecDestroy(cg->exec); if (cg->graph) (void)hipGraphDestroy(cg->graph); delete cg; }
    }
  } closer{g_openCapture};
  CapturedGraph* cg = closer.cg;
  hipError_t e = hipStreamEndCapture(execStream(), &cg->graph);
  closer.streamOpen = false;
  if (e != hipSuccess || cg->graph == nullptr) {
    (void)hipGetLastError();
    ND4J_THROW(std::string("nd4jhipGraphEndCapture: the capture was invalidated (an op waited on the stream or copied synchronously): ") + hipGetErrorString(e));
  }
  // Every call of the capture was one the facade keeps a record of: run the sequence again through the merging pass and
  // keep that recording instead (nothing has executed so far -- a capture only notes launches)
  bool keepPlan = false;
  if (graphFusionEnabled() && !cg->ops.empty() && (int)cg->ops.size() == cg->opCalls) {
    int nFused = 0;
    cg->plan = fuseRecordedOps(cg->ops, nFused);
    keepPlan = true;
    if (nFused > 0) {
      g_captureOpCalls = nullptr;             // the replay re-enters nothing that counts
      hipGraph_t merged = nullptr;
      cg->record = CaptureRecord();
      std::string failure;
      e = hipStreamBeginCapture(execStream(), hipStreamCaptureModeRelaxed);
      if (e == hipSuccess) {
        closer.streamOpen = true;
        std::vector<RecordedOp> keep;
        keep.swap(cg->ops);                   // replayed ops must not be recorded a second time
        fusedAppliedCounter() = 0;
        try { for (auto& step : cg->plan) step(); } catch (std::exception& ex) { failure = ex.what(); } catch (...) { failure = "unknown native error"; }
        cg->fusedApplied = fusedAppliedCounter();
        cg->ops.swap(keep);
        e = hipStreamEndCapture(execStream(), &merged);
        closer.streamOpen = false;
      }
      if (e == hipSuccess && merged != nullptr && failure.empty()) {
        (void)hipGraphDestroy(cg->graph);
        cg->graph = merged;
        cg->fusedOps = nFused;
      } else {
        if (merged) (void)hipGraphDestroy(merged);
        (void)hipGetLastError();
        ND4J_THROW("nd4jhipGraphEndCapture: replaying the recorded ops through the merging pass failed: " + (failure.empty() ? std::string(hipGetErrorString(e)) : failure));
      }
    }
  }
  if (!keepPlan) cg->ops.clear();   // (the plan's steps point into the list)
  e = hipGraphInstantiate(&cg->exec, cg->graph, nullptr, nullptr, 0);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    ND4J_THROW(std::string("nd4jhipGraphEndCapture: hipGraphInstantiate failed: ") + hipGetErrorString(e));
  }
  closer.cg = nullptr;   // handed to the caller
  return cg;
  GUARD_END(nullptr)
}
}  // extern "C"
// Is a rocprofiler tool library attached to this process?  A graph launch under the kernel tracer once ended in a queue
// abort ("AQL packet is malformed") whose cause was never established, so a traced process does not launch graphs:
// nd4jhipGraphLaunch replays the recorded plan kernel by kernel instead (same kernels, same arguments).  The tool is
// found by what loads it: ROCP_TOOL_LIBRARIES or LD_PRELOAD naming it, or the loaded object itself.
static bool nameIsProfilerTool(const char* s) { return s != nullptr && (strstr(s, "rocprofiler-sdk-tool") != nullptr || strstr(s, "librocprofv3") != nullptr); }
static bool profilerToolAttached() {
  const char* tools = getenv("ROCP_TOOL_LIBRARIES");
  if (tools != nullptr && *tools) return true;
  if (nameIsProfilerTool(getenv("LD_PRELOAD"))) return true;
  bool found = false;
  dl_iterate_phdr([](struct dl_phdr_info* info, size_t, void* data) -> int {
    if (nameIsProfilerTool(info->dlpi_name)) { *static_cast<bool*>(data) = true; return 1; }
    return 0;
  }, &found);
  return found;
}
extern "C" {
int nd4jhipProfilerAttached(void) { return profilerToolAttached() ? 1 : 0; }
int nd4jhipGraphLaunch(Nd4jPointer graph) {
  GRAPH_BEGIN
  ND4J_REQUIRE(graph != nullptr, "nd4jhipGraphLaunch: graph is null");
  ND4J_REQUIRE(!captureActive(), "nd4jhipGraphLaunch: a capture is in progress");
  CapturedGraph* cg = static_cast<CapturedGraph*>(graph);
  bool asKernels = g_graphReplayMode == 1 && !cg->plan.empty();
  if (!asKernels) {
    static const bool traced = profilerToolAttached();   // a tool attaches before main(): asked once
    if (traced) {
      ND4J_REQUIRE(!cg->plan.empty(), "nd4jhipGraphLaunch: a rocprofiler tool is attached to this process and this recording has no kernel-by-kernel plan (an op "
                                      "call went unrecorded during its capture); graphs are not launched under the tracer");
      static std::once_flag said;
      if (Environment::get().verbose) std::call_once(said, [] { fprintf(stderr, "nd4j-hip: a rocprofiler tool is attached; recorded graphs are replayed kernel by kernel\n"); });
      asKernels = true;
    }
  }
  if (asKernels) {
    // the merged sequence as ordinary launches: every step prepares and registers its own arrays, as the eager call does
    for (auto& b : cg->record.reads) ND4J_REQUIRE(!b->closed, "nd4jhipGraphLaunch: a buffer the graph reads has been closed");
    for (auto& b : cg->record.writes) ND4J_REQUIRE(!b->closed, "nd4jhipGraphLaunch: a buffer the graph writes has been closed");
    const bool syncWas = Environment::get().syncAfterCustomOp;
    Environment::get().syncAfterCustomOp = false;   // as during the capture: nothing waits inside a step
    fusedAppliedCounter() = 0;
    try { for (auto& step : cg->plan) step(); } catch (...) { Environment::get().syncAfterCustomOp = syncWas; throw; }
    cg->fusedApplied = fusedAppliedCounter();
    Environment::get().syncAfterCustomOp = syncWas;
    return 0;
  }
  // what prepareSpecialUse does per op, for the whole recorded sequence: an input (or a partly written output) whose
  // host copy is newer goes to the device first
  for (auto& b : cg->record.reads) {
    ND4J_REQUIRE(!b->closed, "nd4jhipGraphLaunch: a buffer the graph reads has been closed");
    b->syncToSpecial();
  }
  for (auto& b : cg->record.writes) {
    ND4J_REQUIRE(!b->closed && b->special, "nd4jhipGraphLaunch: a buffer the graph writes has been closed");
    if (!b->isSpecialActual()) b->syncToSpecial();
  }
  HIP_CHECK(hipGraphLaunch(cg->exec, execStream()));
  // ... and what registerSpecialUse does: outputs are now newest on the device
  for (auto& b : cg->record.reads) b->tickReadSpecial();
  for (auto& b : cg->record.writes) b->tickWriteSpecial();
  return 0;
  GUARD_END(1)
}
// Host-side audit of a recording: every kernel node's block size, dynamic LDS request and grid against what the runtime
// reports for that function (hipFuncGetAttributes) and for the device.  Launches nothing.  Returns the number of nodes
// that break a limit (their description goes to the error slot), 0 for a clean graph, -1 when the graph cannot be walked.
int nd4jhipGraphAudit(Nd4jPointer graph) {
  GRAPH_BEGIN
  ND4J_REQUIRE(graph != nullptr, "nd4jhipGraphAudit: graph is null");
  CapturedGraph* cg = static_cast<CapturedGraph*>(graph);
  size_t n = 0;
  HIP_CHECK(hipGraphGetNodes(cg->graph, nullptr, &n));
  std::vector<hipGraphNode_t> nodes(n);
  if (n) HIP_CHECK(hipGraphGetNodes(cg->graph, nodes.data(), &n));
  int dev = 0;
  HIP_CHECK(hipGetDevice(&dev));
  hipDeviceProp_t prop;
  HIP_CHECK(hipGetDeviceProperties(&prop, dev));
  int bad = 0, kernels = 0;
  std::string report;
  for (size_t i = 0; i < n; i++) {
    hipGraphNodeType type;
    HIP_CHECK(hipGraphNodeGetType(nodes[i], &type));
    if (type != hipGraphNodeTypeKernel) continue;
    kernels++;
    hipKernelNodeParams kp;
    HIP_CHECK(hipGraphKernelNodeGetParams(nodes[i], &kp));
    hipFuncAttributes fa;
    std::string why;
    if (hipFuncGetAttributes(&fa, kp.func) != hipSuccess) { (void)hipGetLastError(); why = "hipFuncGetAttributes failed"; }
    else {
      const long long threads = (long long)kp.blockDim.x * kp.blockDim.y * kp.blockDim.z;
      if (threads <= 0 || threads > fa.maxThreadsPerBlock) why += " block of " + std::to_string(threads) + " threads (limit " + std::to_string(fa.maxThreadsPerBlock) + ")";
      if ((long long)kp.sharedMemBytes > (long long)fa.maxDynamicSharedSizeBytes) why += " dynamic LDS " + std::to_string(kp.sharedMemBytes) + " B (granted " + std::to_string(fa.maxDynamicSharedSizeBytes) + ")";
      if ((long long)kp.sharedMemBytes + (long long)fa.sharedSizeBytes > (long long)prop.sharedMemPerBlock && (long long)kp.sharedMemBytes + (long long)fa.sharedSizeBytes > (long long)prop.maxSharedMemoryPerMultiProcessor)
        why += " LDS total " + std::to_string((long long)kp.sharedMemBytes + (long long)fa.sharedSizeBytes) + " B beyond the CU's";
      if (kp.gridDim.x == 0 || kp.gridDim.y == 0 || kp.gridDim.z == 0 || kp.gridDim.y > 65535u || kp.gridDim.z > 65535u) why += " grid " + std::to_string(kp.gridDim.x) + "x" + std::to_string(kp.gridDim.y) + "x" + std::to_string(kp.gridDim.z);
      if (kp.kernelParams == nullptr && kp.extra == nullptr) why += " no kernel arguments recorded";
    }
    if (!why.empty()) { bad++; report += "node " + std::to_string(i) + ":" + why + "; "; }
  }
  if (bad) errorRef().set(1, "nd4jhipGraphAudit: " + std::to_string(bad) + " of " + std::to_string(kernels) + " kernel nodes: " + report);
  return bad;
  GUARD_END(-1)
}
int nd4jhipGraphFusedOps(Nd4jPointer graph) { return graph ? static_cast<CapturedGraph*>(graph)->fusedOps : 0; }
int nd4jhipGraphFusedApplied(Nd4jPointer graph) { return graph ? static_cast<CapturedGraph*>(graph)->fusedApplied : 0; }
void nd4jhipSetGraphReplayMode(int mode) { g_graphReplayMode = mode == 1 ? 1 : 0; }
int nd4jhipGetGraphReplayMode(void) { return g_graphReplayMode; }
void nd4jhipGraphDestroy(Nd4jPointer graph) {
  if (!graph) return;
  CapturedGraph* cg = static_cast<CapturedGraph*>(graph);
  if (cg->exec) (void)hipGraphExecDestroy(cg->exec);
  if (cg->graph) (void)hipGraphDestroy(cg->graph);
  delete cg;
}
const char* nd4jhipLastGemmKernel(void) { return lastGemmKernel(); }
int nd4jhipAttentionBlockOrder(int batchEntries, int queryTiles, int keyTilesPerQueryTile, int residentBlocksPerCu, unsigned short* items) {
  if (items == nullptr) return 0;
  return attentionBlockOrder(batchEntries, queryTiles, keyTilesPerQueryTile, residentBlocksPerCu, items);
}

// execReduceSame (full reduction of a dense array) for callers that cannot allocate: plain device pointers in, one
// element out, partials in a fixed device array.  No hipMalloc / hipFree on any path, the error paths included.
int nd4jhipReduceSameScalarNoAlloc(Nd4jPointer stream, int opNum, int dataType, const void* dX, Nd4jLong length, void* dZ) {
  OP_BEGIN(nullptr)
  LaunchContext* lc = LaunchContext::ifReady();
  ND4J_REQUIRE(lc != nullptr, "nd4jhipReduceSameScalarNoAlloc: call initializeDevicesAndFunctions first (initialisation allocates, this call must not)");
  // between nd4jhipGraphBeginCapture and End a null stream is the capturing stream itself: the launches become nodes of
  // that graph (the call leaves no record for the kernel-by-kernel plan, so such a recording replays as a graph only)
  ND4J_REQUIRE(dX != nullptr && dZ != nullptr, "nd4jhipReduceSameScalarNoAlloc: null device pointer");
  const DataType dt = (DataType)dataType;
  ND4J_REQUIRE(isFloatType(dt), "nd4jhipReduceSameScalarNoAlloc: FLOAT, DOUBLE, HALF or BFLOAT16 arrays only");
  ND4J_REQUIRE((reinterpret_cast<uintptr_t>(dX) % sizeOf(dt)) == 0 && (reinterpret_cast<uintptr_t>(dZ) % sizeOf(dt)) == 0, "nd4jhipReduceSameScalarNoAlloc: misaligned pointer");
  hipStream_t st = stream ? *reinterpret_cast<hipStream_t*>(stream) : lc->execStream;
  launchReduceScalarNoAlloc(st, reduceSameKind(opNum), dt, dX, length, dZ);
  return 0;
  GUARD_END(1)
}
const char* nd4jhipBuildInfo(void) { return "nd4j-hip gfx950 (hand-written HIP kernels; no CPU fallback)"; }

}  // extern "C"
