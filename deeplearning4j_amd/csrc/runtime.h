// Host runtime behind the NativeOps boundary: error slot, launch context, data buffers with
// host/device coherence stamps, array handles, descriptor/TAD caches and the per-op context.
#pragma once
#include <hip/hip_runtime.h>

#include <atomic>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <map>
#include <memory>
#include <mutex>
#include <stdexcept>
#include <string>
#include <vector>

#include "types.h"

namespace nd4jhip {

// ---- errors ------------------------------------------------------------------------------------
// Facade functions catch exceptions and park {code, message} here; the caller polls
// lastErrorCode()/lastErrorMessage() (reference convention: legacy/cpu/NativeOps.cpp:1118-1121).
struct ErrorReference {
  std::mutex lock;
  int code = 0;
  std::string message;
  void set(int c, const std::string& m);
  void clear();
};
ErrorReference& errorRef();

[[noreturn]] void throwError(const std::string& msg);
#define ND4J_THROW(msg) ::nd4jhip::throwError(std::string(msg))
#define ND4J_REQUIRE(cond, msg) \
  do {                          \
    if (!(cond)) ::nd4jhip::throwError(std::string(msg)); \
  } while (0)
#define HIP_CHECK(expr)                                                                              \
  do {                                                                                               \
    hipError_t _e = (expr);                                                                          \
    if (_e != hipSuccess)                                                                            \
      ::nd4jhip::throwError(std::string(#expr) + " failed: " + hipGetErrorString(_e));               \
  } while (0)

// ---- launch context -------------------------------------------------------------------------------
// One execution stream and one copy stream (default priority), a device scratch area for cross-block
// partials and a pinned scalar slot (reference: execution/cuda/ContextBuffers.cu:129-136).
struct LaunchContext {
  hipStream_t execStream = nullptr;
  hipStream_t copyStream = nullptr;
  void* reductionBuffer = nullptr;   // device, REDUCTION_BYTES
  void* allocationBuffer = nullptr;  // device, ALLOCATION_BYTES
  void* scalarBuffer = nullptr;      // pinned host, 256 B
  hipEvent_t bridgeIn = nullptr, bridgeOut = nullptr;   // order a caller-owned stream against execStream
  int deviceId = 0;
  bool ready = false;
  static constexpr size_t REDUCTION_BYTES = 8u << 20;
  static constexpr size_t ALLOCATION_BYTES = 8u << 20;
  // Grow-only device scratch for ops whose temporaries are as large as their operands (the attention composition's logits
  // and weights, dense copies of masks).  It only ever grows, and only outside a stream capture: an op that fits what is
  // there neither allocates nor waits, and whatever the previous op left in it is no longer read once this op's first
  // kernel starts (one stream, one op at a time).  Call with the sum of what the op will carve out of it.
  void* workspace(size_t bytes);
  void* workspaceBuffer = nullptr;
  size_t workspaceBytes = 0;
  void init();
  static LaunchContext* defaultContext();
  static LaunchContext* ifReady();   // the default context if it has been initialised, else null (never allocates)
};
bool deviceAvailable();

// ---- data buffer ----------------------------------------------------------------------------------
// Host ("primary") + device ("special") storage with four monotonically increasing stamps; which
// side is current follows array/cuda/DataBuffer.cu:597-606 of the reference.
struct DataBuffer {
  void* primary = nullptr;
  void* special = nullptr;
  size_t lenBytes = 0;
  DataType dtype = FLOAT32;
  bool ownsPrimary = false, ownsSpecial = false;
  bool pinnedPrimary = false;   // primary came from hipHostMalloc (owned buffers of 1 MiB and more)
  bool closed = false;
  int deviceId = 0;
  std::atomic<LongType> counter{0};
  LongType writePrimary = 0, writeSpecial = 0, readPrimary = 0, readSpecial = 0;

  DataBuffer(size_t bytes, DataType dt, bool allocBoth);
  DataBuffer(void* prim, void* spec, size_t bytes, DataType dt);  // external, not owned
  ~DataBuffer();
  LongType numElements() const { return sizeOf(dtype) ? (LongType)(lenBytes / sizeOf(dtype)) : 0; }
  void allocatePrimary();
  void releasePrimary();
  void allocateSpecial();
  bool isPrimaryActual() const { return writePrimary > writeSpecial || readPrimary > writeSpecial; }
  bool isSpecialActual() const { return writeSpecial > writePrimary || readSpecial > writePrimary; }
  void tickWritePrimary() { writePrimary = ++counter; }
  void tickWriteSpecial() { writeSpecial = ++counter; }
  void tickReadPrimary() { readPrimary = ++counter; }
  void tickReadSpecial() { readSpecial = ++counter; }
  void syncToSpecial(bool force = false);
  void syncToPrimary(bool force = false);
  void expand(size_t newBytes);
  void close();
};

// What Java sees as OpaqueDataBuffer (array/InteropDataBuffer.h:32-118): a handle onto a shared
// DataBuffer plus a byte offset for views.
struct InteropDataBuffer {
  std::shared_ptr<DataBuffer> db;
  size_t offsetBytes = 0;
  void* primary() const { return db && db->primary ? (char*)db->primary + offsetBytes : nullptr; }
  void* special() const { return db && db->special ? (char*)db->special + offsetBytes : nullptr; }
};

// ---- array handle -------------------------------------------------------------------------------
// (DataBuffer, shapeInfo, element offset); does not own the buffer (legacy/impl/NativeOpsHelpers_Arrays.cpp:149-193).
struct NDArray {
  std::shared_ptr<DataBuffer> buf;
  size_t bufOffsetBytes = 0;  // offset of the InteropDataBuffer view
  std::vector<LongType> si;   // private copy of the descriptor
  LongType offset = 0;        // element offset of the array view

  const LongType* shapeInfo() const { return si.data(); }
  int rankOf() const { return shape::rank(si.data()); }
  LongType sizeAt(int d) const { int r = rankOf(); if (d < 0) d += r; return shape::shapeOf(si.data())[d]; }
  LongType strideAt(int d) const { int r = rankOf(); if (d < 0) d += r; return shape::strideOf(si.data())[d]; }
  LongType lengthOf() const { return shape::length(si.data()); }
  DataType dataType() const { return shape::dataType(si.data()); }
  bool isEmpty() const { return shape::isEmpty(si.data()); }
  char ordering() const { return shape::order(si.data()); }
  // pointers to the first element of the view (offset applied exactly once)
  void* buffer() const;
  void* specialBuffer() const;
  template <typename T> T* hostAs() const { return reinterpret_cast<T*>(buffer()); }
};

// ---- kernels that ask for more dynamic LDS than the default limit -----------------------------------------------------
// Such a kernel needs one hipFuncSetAttribute call before its first launch.  Every instantiation the dispatchers can pick
// registers its setter when the library is loaded (DynLds below), and the launch context runs all of them when it is
// created, so that no attribute call can fire for the first time between the Begin and End of a stream capture.
void registerKernelAttribute(void (*apply)());
void applyKernelAttributes();   // runs the setters registered so far that have not run yet (the device must be current)
template <auto Kern, int BYTES>
struct DynLds {
  static bool granted_;
  static const bool registered_;
  static void apply() {
    granted_ = hipFuncSetAttribute(reinterpret_cast<const void*>(Kern), hipFuncAttributeMaxDynamicSharedMemorySize, BYTES) == hipSuccess;
    if (!granted_) (void)hipGetLastError();
  }
  // did the device grant this kernel BYTES of dynamic LDS
  static bool granted() {
    (void)registered_;          // forces the registration of this instantiation at load time
    applyKernelAttributes();    // a no-op once the launch context exists
    return granted_;
  }
};
template <auto Kern, int BYTES> bool DynLds<Kern, BYTES>::granted_ = false;
template <auto Kern, int BYTES> const bool DynLds<Kern, BYTES>::registered_ = (registerKernelAttribute(&DynLds<Kern, BYTES>::apply), true);

// ---- stream capture ---------------------------------------------------------------------------------
// While a capture is open, ops record their kernels instead of running them, and prepare/registerSpecialUse note which
// buffers the recorded kernels read and write, so that a replay can bring inputs up to date and stamp outputs.
struct CaptureRecord {
  std::vector<std::shared_ptr<DataBuffer>> reads, writes;
  void noteRead(const std::shared_ptr<DataBuffer>& b);
  void noteWrite(const std::shared_ptr<DataBuffer>& b);
};
bool captureActive();
CaptureRecord* activeCapture();
void setActiveCapture(CaptureRecord* rec);   // null: no capture open

// prepareSpecialUse / registerSpecialUse (array/cuda/NDArray.cu:331-357)
void prepareSpecialUse(std::initializer_list<NDArray*> writes, std::initializer_list<NDArray*> reads);
void registerSpecialUse(std::initializer_list<NDArray*> writes, std::initializer_list<NDArray*> reads);
void prepareSpecialUse(const std::vector<NDArray*>& writes, const std::vector<NDArray*>& reads);
void registerSpecialUse(const std::vector<NDArray*>& writes, const std::vector<NDArray*>& reads);

// ---- descriptor cache ---------------------------------------------------------------------------
struct ConstantShapeBuffer {
  std::vector<LongType> host;
  LongType* device = nullptr;
  const LongType* primary() const { return host.data(); }
  const LongType* special();
};
ConstantShapeBuffer* cachedShapeBuffer(const LongType* shapeInfo);
std::vector<LongType> makeShapeInfo(DataType dt, char order, const std::vector<LongType>& shape,
                                    const LongType* strides = nullptr, LongType extraFlags = 0);
std::vector<LongType> scalarShapeInfo(DataType dt);

// ---- TAD pack (helpers/cpu/TadCalculator.cpp:25-100) ----------------------------------------------
struct TadPack {
  ConstantShapeBuffer* tadShape = nullptr;
  std::vector<LongType> offsets;
  LongType* deviceOffsets = nullptr;
  LongType numTads = 0;
  const LongType* specialOffsets();
};
TadPack* tadForDimensions(const LongType* shapeInfo, const LongType* dims, int ndims);

struct ShapeList {
  std::vector<ConstantShapeBuffer*> shapes;
};

// ---- per-op context (graph/Context.h:43-291) ------------------------------------------------------
struct Context {
  int nodeId = 0;
  std::vector<NDArray*> inputs, outputs;  // borrowed
  std::vector<double> tArgs;
  std::vector<LongType> iArgs;
  std::vector<bool> bArgs;
  std::vector<DataType> dArgs;
  bool inplace = false;
  bool helpersAllowed = true;
  bool shapeFunctionOverride = false;
  int execMode = 0;
  LongType rootSeed = 0, nodeSeed = 0;
  // what setGraphContextCudaContext handed in (graph/Context.h setCudaContext): pointer to the caller's stream, its scratch
  void* callerStream = nullptr;
  void* callerReduction = nullptr;
  void* callerAllocation = nullptr;
  int width() const { return (int)inputs.size(); }
  NDArray* input(int i) const;
  NDArray* output(int i) const;
};

// ---- environment ----------------------------------------------------------------------------------
struct Environment {
  bool verbose = false, debug = false;
  // execCustomOp2 synchronises the stream before returning, as the reference's device backend does
  // (legacy/cuda/NativeOps.cu:118); the decode harness may switch this off and synchronise once per step.
  bool syncAfterCustomOp = true;
  int maxThreads = 1;
  static Environment& get();
};

// one element of host memory, widened to double (float types only)
inline double hostValueAsDouble(const void* p, DataType dt) {
  switch (dt) {
    case DOUBLE: return *static_cast<const double*>(p);
    case FLOAT32: return *static_cast<const float*>(p);
    case BFLOAT16: { const uint32_t b = (uint32_t)*static_cast<const uint16_t*>(p) << 16; float f; std::memcpy(&f, &b, 4); return f; }
    case HALF: {
      const uint16_t h = *static_cast<const uint16_t*>(p);
      const int e = (h >> 10) & 31, m = h & 1023;
      double v = e == 0 ? std::ldexp((double)m, -24) : e == 31 ? (m ? NAN : INFINITY) : std::ldexp((double)(m | 1024), e - 25);
      return (h & 0x8000) ? -v : v;
    }
    default: ND4J_THROW("a floating point value is required here");
  }
}

}  // namespace nd4jhip
