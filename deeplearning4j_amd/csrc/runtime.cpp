#include "runtime.h"

#include <cstdlib>
#include <cstring>

namespace nd4jhip {

// ---- errors ------------------------------------------------------------------------------------
void ErrorReference::set(int c, const std::string& m) {
  std::lock_guard<std::mutex> g(lock);
  code = c;
  message = m;
}
void ErrorReference::clear() {
  std::lock_guard<std::mutex> g(lock);
  code = 0;
  message.clear();
}
ErrorReference& errorRef() {
  static ErrorReference r;
  return r;
}
void throwError(const std::string& msg) { throw std::runtime_error(msg); }

Environment& Environment::get() {
  static Environment e = [] {
    Environment v;
    if (const char* s = getenv("ND4JHIP_VERBOSE")) v.verbose = atoi(s) != 0;
    if (const char* s = getenv("ND4JHIP_SYNC_CUSTOM_OPS")) v.syncAfterCustomOp = atoi(s) != 0;
    return v;
  }();
  return e;
}

// ---- shape helpers -------------------------------------------------------------------------------
namespace shape {
LongType flagForDataType(DataType t) {
  switch (t) {
    case HALF: return ARRAY_HALF;
    case BFLOAT16: return ARRAY_BHALF;
    case FLOAT32: return ARRAY_FLOAT;
    case DOUBLE: return ARRAY_DOUBLE;
    case INT8: return ARRAY_CHAR;
    case INT16: return ARRAY_SHORT;
    case INT32: return ARRAY_INT;
    case INT64: return ARRAY_LONG;
    case BOOL: return ARRAY_BOOL;
    case UINT8: return ARRAY_CHAR | ARRAY_UNSIGNED;
    case UINT16: return ARRAY_SHORT | ARRAY_UNSIGNED;
    case UINT32: return ARRAY_INT | ARRAY_UNSIGNED;
    case UINT64: return ARRAY_LONG | ARRAY_UNSIGNED;
    default: return 0;
  }
}
DataType dataType(const LongType* si) {
  LongType e = extra(si);
  if (e & ARRAY_UNSIGNED) {
    if (e & ARRAY_CHAR) return UINT8;
    if (e & ARRAY_SHORT) return UINT16;
    if (e & ARRAY_INT) return UINT32;
    if (e & ARRAY_LONG) return UINT64;
    return UNKNOWN;
  }
  if (e & ARRAY_FLOAT) return FLOAT32;
  if (e & ARRAY_DOUBLE) return DOUBLE;
  if (e & ARRAY_HALF) return HALF;
  if (e & ARRAY_BHALF) return BFLOAT16;
  if (e & ARRAY_BOOL) return BOOL;
  if (e & ARRAY_CHAR) return INT8;
  if (e & ARRAY_SHORT) return INT16;
  if (e & ARRAY_INT) return INT32;
  if (e & ARRAY_LONG) return INT64;
  return UNKNOWN;
}
}  // namespace shape

std::vector<LongType> makeShapeInfo(DataType dt, char order, const std::vector<LongType>& shp, const LongType* strides,
                                    LongType extraFlags) {
  int r = (int)shp.size();
  std::vector<LongType> si(shape::shapeInfoLength(r), 0);
  LongType flags = (extraFlags & ~ARRAY_ALL_DTYPE_BITS) | shape::flagForDataType(dt);
  if (r == 0) {
    si[0] = 0; si[1] = 0; si[2] = 1; si[3] = flags; si[4] = 1; si[5] = order ? order : 'c';
    return si;
  }
  si[0] = r;
  bool hasZero = false;
  for (int i = 0; i < r; i++) { si[1 + i] = shp[i]; if (shp[i] == 0) hasZero = true; }
  if (strides) {
    for (int i = 0; i < r; i++) si[1 + r + i] = strides[i];
  } else if (order == 'f') {
    LongType s = 1;
    for (int i = 0; i < r; i++) { si[1 + r + i] = s; s *= shp[i] ? shp[i] : 1; }
  } else {
    LongType s = 1;
    for (int i = r - 1; i >= 0; i--) { si[1 + r + i] = s; s *= shp[i] ? shp[i] : 1; }
  }
  if (hasZero) flags |= ARRAY_EMPTY;
  si[2 * r + 1] = flags;
  // ews: 1 when the strides are the dense strides of `order`, else 0
  LongType ews = 1;
  if (strides) {
    LongType s = 1;
    if (order == 'f') { for (int i = 0; i < r; i++) { if (shp[i] != 1 && strides[i] != s) ews = 0; s *= shp[i]; } }
    else { for (int i = r - 1; i >= 0; i--) { if (shp[i] != 1 && strides[i] != s) ews = 0; s *= shp[i]; } }
  }
  si[2 * r + 2] = ews;
  si[2 * r + 3] = order ? order : 'c';
  return si;
}
std::vector<LongType> scalarShapeInfo(DataType dt) { return makeShapeInfo(dt, 'c', {}); }

// ---- launch context -------------------------------------------------------------------------------
bool deviceAvailable() {
  static const bool available = [] {
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess) { (void)hipGetLastError(); n = 0; }
    return n > 0;
  }();
  return available;
}

namespace {
struct AttrRegistry {
  std::mutex m;
  std::vector<void (*)()> setters;
  size_t applied = 0;
};
AttrRegistry& attrRegistry() { static AttrRegistry* r = new AttrRegistry(); return *r; }   // outlives every static that registers
}
void registerKernelAttribute(void (*apply)()) {
  AttrRegistry& r = attrRegistry();
  std::lock_guard<std::mutex> g(r.m);
  r.setters.push_back(apply);
}
void applyKernelAttributes() {
  AttrRegistry& r = attrRegistry();
  std::lock_guard<std::mutex> g(r.m);
  while (r.applied < r.setters.size()) r.setters[r.applied++]();
}

void LaunchContext::init() {
  if (ready) return;
  if (!deviceAvailable())
    ND4J_THROW("nd4j-hip: no HIP device is visible; this backend has no CPU fallback");
  HIP_CHECK(hipGetDevice(&deviceId));
  HIP_CHECK(hipStreamCreateWithFlags(&execStream, hipStreamNonBlocking));
  HIP_CHECK(hipStreamCreateWithFlags(&copyStream, hipStreamNonBlocking));
  HIP_CHECK(hipMalloc(&reductionBuffer, REDUCTION_BYTES));
  HIP_CHECK(hipMalloc(&allocationBuffer, ALLOCATION_BYTES));
  HIP_CHECK(hipHostMalloc(&scalarBuffer, 256, hipHostMallocDefault));
  HIP_CHECK(hipEventCreateWithFlags(&bridgeIn, hipEventDisableTiming));
  HIP_CHECK(hipEventCreateWithFlags(&bridgeOut, hipEventDisableTiming));
  applyKernelAttributes();
  ready = true;
}
void* LaunchContext::workspace(size_t bytes) {
  if (bytes <= workspaceBytes) return workspaceBuffer;
  ND4J_REQUIRE(!captureActive(), "this op needs " + std::to_string(bytes) + " bytes of device scratch and " + std::to_string(workspaceBytes) +
                                     " are allocated: run it once outside the capture (allocating would invalidate the recording)");
  HIP_CHECK(hipStreamSynchronize(execStream));   // kernels of earlier ops may still read the old block
  if (workspaceBuffer) (void)hipFree(workspaceBuffer);
  workspaceBuffer = nullptr; workspaceBytes = 0;
  const size_t want = ((bytes + bytes / 4) + 0xfffffu) & ~(size_t)0xfffffu;   // a quarter of headroom, whole MiB
  HIP_CHECK(hipMalloc(&workspaceBuffer, want));
  workspaceBytes = want;
  return workspaceBuffer;
}
static LaunchContext g_defaultContext;
static std::mutex g_defaultContextMutex;
LaunchContext* LaunchContext::defaultContext() {
  std::lock_guard<std::mutex> g(g_defaultContextMutex);
  g_defaultContext.init();
  return &g_defaultContext;
}
LaunchContext* LaunchContext::ifReady() {
  std::lock_guard<std::mutex> g(g_defaultContextMutex);
  return g_defaultContext.ready ? &g_defaultContext : nullptr;
}

// ---- data buffer ----------------------------------------------------------------------------------
DataBuffer::DataBuffer(size_t bytes, DataType dt, bool allocBoth) : lenBytes(bytes), dtype(dt) {
  allocatePrimary();
  if (allocBoth) allocateSpecial();
  // a freshly allocated buffer counts as written on the host
  writePrimary = ++counter;
}
DataBuffer::DataBuffer(void* prim, void* spec, size_t bytes, DataType dt)
    : primary(prim), special(spec), lenBytes(bytes), dtype(dt) {
  if (prim) writePrimary = ++counter;
  if (spec && !prim) writeSpecial = ++counter;
}
DataBuffer::~DataBuffer() { close(); }
// Host buffers of this size and more are page-locked when a device is present (as the device backend's own host
// allocations are, legacy/cuda/NativeOps.cu:1158-1168 mallocHost): the copies of syncToSpecial / syncToPrimary then run as
// one DMA transfer at the link's rate instead of being staged through the runtime's bounce buffers.  Smaller ones stay
// pageable, a page-locked allocation costs more than their copy.  ND4JHIP_PINNED_MIN_BYTES overrides the size (0 = never).
static size_t pinnedMinBytes() {
  static const size_t v = [] {
    const char* e = getenv("ND4JHIP_PINNED_MIN_BYTES");
    if (!e || !*e) return (size_t)1 << 20;
    const unsigned long long n = strtoull(e, nullptr, 10);
    return n == 0 ? (size_t)-1 : (size_t)n;
  }();
  return v;
}
void DataBuffer::allocatePrimary() {
  if (primary || lenBytes == 0) return;
  void* p = nullptr;
  if (lenBytes >= pinnedMinBytes() && deviceAvailable()) {
    LaunchContext::defaultContext();
    if (hipHostMalloc(&p, lenBytes, hipHostMallocDefault) == hipSuccess) pinnedPrimary = true;
    else { (void)hipGetLastError(); p = nullptr; }   // no page-locked memory left: a pageable buffer does the same job, slower
  }
  if (!p && posix_memalign(&p, 64, lenBytes) != 0) ND4J_THROW("DataBuffer: host allocation failed");
  memset(p, 0, lenBytes);
  primary = p;
  ownsPrimary = true;
}
void DataBuffer::releasePrimary() {
  if (ownsPrimary && primary) {
    if (pinnedPrimary) (void)hipHostFree(primary);
    else free(primary);
  }
  primary = nullptr;
  ownsPrimary = pinnedPrimary = false;
}
void DataBuffer::allocateSpecial() {
  if (special || lenBytes == 0) return;
  LaunchContext::defaultContext();
  HIP_CHECK(hipMalloc(&special, lenBytes));
  ownsSpecial = true;
}
void DataBuffer::syncToSpecial(bool force) {
  // array/cuda/DataBuffer.cu:399-413
  if (lenBytes == 0) return;
  if (!primary) { if (!special) allocateSpecial(); return; }
  if (!force && special && isSpecialActual()) return;
  if (!special) allocateSpecial();
  auto lc = LaunchContext::defaultContext();
  HIP_CHECK(hipMemcpyAsync(special, primary, lenBytes, hipMemcpyHostToDevice, lc->execStream));
  // the caller may rewrite the host memory as soon as this returns (array/cuda/DataBuffer.cu:399-413 copies synchronously)
  HIP_CHECK(hipStreamSynchronize(lc->execStream));
  readSpecial = ++counter;  // device copy is current; the host copy stays current too
}
void DataBuffer::syncToPrimary(bool force) {
  // array/cuda/DataBuffer.cu:367-395
  if (lenBytes == 0 || !special) return;
  if (!force && isPrimaryActual() && primary) return;
  if (!primary) allocatePrimary();
  auto lc = LaunchContext::defaultContext();
  HIP_CHECK(hipStreamSynchronize(lc->execStream));
  HIP_CHECK(hipMemcpy(primary, special, lenBytes, hipMemcpyDeviceToHost));
  readPrimary = ++counter;  // host copy is current; the device copy stays current too
}
void DataBuffer::expand(size_t newBytes) {
  if (newBytes <= lenBytes) return;
  if (primary) {
    void* const old = primary;
    const bool oldOwned = ownsPrimary, oldPinned = pinnedPrimary;
    const size_t oldBytes = lenBytes;
    primary = nullptr; ownsPrimary = pinnedPrimary = false;
    lenBytes = newBytes;
    allocatePrimary();   // zero-filled, page-locked from the same size on
    lenBytes = oldBytes;
    memcpy(primary, old, oldBytes);
    if (oldOwned) { if (oldPinned) (void)hipHostFree(old); else free(old); }
  }
  if (special) {
    void* d = nullptr;
    HIP_CHECK(hipMalloc(&d, newBytes));
    auto lc = LaunchContext::defaultContext();
    HIP_CHECK(hipMemsetAsync(d, 0, newBytes, lc->execStream));
    HIP_CHECK(hipMemcpyAsync(d, special, lenBytes, hipMemcpyDeviceToDevice, lc->execStream));
    HIP_CHECK(hipStreamSynchronize(lc->execStream));
    if (ownsSpecial) (void)hipFree(special);
    special = d;
    ownsSpecial = true;
  }
  lenBytes = newBytes;
}
void DataBuffer::close() {
  if (closed) return;
  closed = true;
  releasePrimary();
  if (ownsSpecial && special) (void)hipFree(special);
  special = nullptr;
}

// ---- stream capture ---------------------------------------------------------------------------------
static std::atomic<CaptureRecord*> g_capture{nullptr};
bool captureActive() { return g_capture.load(std::memory_order_acquire) != nullptr; }
CaptureRecord* activeCapture() { return g_capture.load(std::memory_order_acquire); }
void setActiveCapture(CaptureRecord* rec) { g_capture.store(rec, std::memory_order_release); }
static void noteUnique(std::vector<std::shared_ptr<DataBuffer>>& v, const std::shared_ptr<DataBuffer>& b) {
  for (auto& e : v) if (e.get() == b.get()) return;
  v.push_back(b);
}
void CaptureRecord::noteRead(const std::shared_ptr<DataBuffer>& b) { noteUnique(reads, b); }
void CaptureRecord::noteWrite(const std::shared_ptr<DataBuffer>& b) { noteUnique(writes, b); }

// ---- array handle -------------------------------------------------------------------------------
void* NDArray::buffer() const {
  if (!buf || !buf->primary) return nullptr;
  return (char*)buf->primary + bufOffsetBytes + (size_t)offset * sizeOf(dataType());
}
void* NDArray::specialBuffer() const {
  if (!buf || !buf->special) return nullptr;
  return (char*)buf->special + bufOffsetBytes + (size_t)offset * sizeOf(dataType());
}

template <typename W, typename R>
static void prepareImpl(const W& writes, const R& reads) {
  for (NDArray* a : reads) if (a && a->buf) a->buf->syncToSpecial();
  for (NDArray* a : writes) {
    if (!a || !a->buf) continue;
    // an output that covers its whole buffer is simply overwritten; a view of a larger buffer must
    // first bring the untouched part up to date on the device
    bool whole = (size_t)a->lengthOf() * sizeOf(a->dataType()) >= a->buf->lenBytes;
    if (whole) a->buf->allocateSpecial();
    else if (!a->buf->special || !a->buf->isSpecialActual()) a->buf->syncToSpecial();
  }
}
template <typename W, typename R>
static void registerImpl(const W& writes, const R& reads) {
  for (NDArray* a : reads) if (a && a->buf) a->buf->tickReadSpecial();
  for (NDArray* a : writes) if (a && a->buf) a->buf->tickWriteSpecial();
  if (CaptureRecord* rec = activeCapture()) {
    for (NDArray* a : reads) if (a && a->buf) rec->noteRead(a->buf);
    for (NDArray* a : writes) if (a && a->buf) rec->noteWrite(a->buf);
  }
}
void prepareSpecialUse(std::initializer_list<NDArray*> w, std::initializer_list<NDArray*> r) { prepareImpl(w, r); }
void registerSpecialUse(std::initializer_list<NDArray*> w, std::initializer_list<NDArray*> r) { registerImpl(w, r); }
void prepareSpecialUse(const std::vector<NDArray*>& w, const std::vector<NDArray*>& r) { prepareImpl(w, r); }
void registerSpecialUse(const std::vector<NDArray*>& w, const std::vector<NDArray*>& r) { registerImpl(w, r); }

// ---- descriptor cache ---------------------------------------------------------------------------
const LongType* ConstantShapeBuffer::special() {
  static std::mutex m;
  std::lock_guard<std::mutex> g(m);
  if (!device) {
    HIP_CHECK(hipMalloc((void**)&device, host.size() * sizeof(LongType)));
    HIP_CHECK(hipMemcpy(device, host.data(), host.size() * sizeof(LongType), hipMemcpyHostToDevice));
  }
  return device;
}
ConstantShapeBuffer* cachedShapeBuffer(const LongType* si) {
  static std::map<std::vector<LongType>, std::unique_ptr<ConstantShapeBuffer>> cache;
  static std::mutex m;
  ND4J_REQUIRE(si != nullptr, "shape cache: shapeInfo is null");
  int r = shape::rank(si);
  ND4J_REQUIRE(r >= 0 && r <= MAX_RANK, "shape cache: rank out of range");
  std::vector<LongType> key(si, si + shape::shapeInfoLength(r));
  std::lock_guard<std::mutex> g(m);
  auto it = cache.find(key);
  if (it != cache.end()) return it->second.get();
  auto b = std::make_unique<ConstantShapeBuffer>();
  b->host = key;
  auto* raw = b.get();
  cache.emplace(std::move(key), std::move(b));
  return raw;
}

// ---- TAD pack -------------------------------------------------------------------------------------
const LongType* TadPack::specialOffsets() {
  static std::mutex m;
  std::lock_guard<std::mutex> g(m);
  if (!deviceOffsets && !offsets.empty()) {
    HIP_CHECK(hipMalloc((void**)&deviceOffsets, offsets.size() * sizeof(LongType)));
    HIP_CHECK(hipMemcpy(deviceOffsets, offsets.data(), offsets.size() * sizeof(LongType), hipMemcpyHostToDevice));
  }
  return deviceOffsets;
}

TadPack* tadForDimensions(const LongType* si, const LongType* dims, int ndims) {
  static std::map<std::pair<std::vector<LongType>, std::vector<LongType>>, std::unique_ptr<TadPack>> cache;
  static std::mutex m;
  ND4J_REQUIRE(si != nullptr, "tadForDimensions: shapeInfo is null");
  ND4J_REQUIRE(!shape::isEmpty(si), "Cannot create TADs for empty array");
  int r = shape::rank(si);
  std::vector<LongType> nd;
  for (int i = 0; i < ndims; i++) {
    LongType d = dims[i] < 0 ? dims[i] + r : dims[i];
    ND4J_REQUIRE(d >= 0 && d < r, "tadForDimensions: dimension out of range");
    nd.push_back(d);
  }
  std::vector<LongType> key(si, si + shape::shapeInfoLength(r));
  std::lock_guard<std::mutex> g(m);
  auto it = cache.find({key, nd});
  if (it != cache.end()) return it->second.get();

  std::vector<bool> keep(r, false);
  for (auto d : nd) keep[d] = true;
  int nk = 0;
  for (int i = 0; i < r; i++) nk += keep[i];
  auto pack = std::make_unique<TadPack>();
  DataType dt = shape::dataType(si);
  if (nk == 0 || nk == r) {
    // all or nothing: scalar TADs with offsets 0..len-1 (TadCalculator.cpp:46-63)
    LongType n = shape::length(si);
    auto s = scalarShapeInfo(dt);
    pack->tadShape = cachedShapeBuffer(s.data());
    pack->offsets.resize(n);
    for (LongType i = 0; i < n; i++) pack->offsets[i] = i;
    pack->numTads = n;
  } else {
    std::vector<LongType> tshape, tstride, oshape, ostride;
    for (int i = 0; i < r; i++) {
      if (keep[i]) { tshape.push_back(shape::shapeOf(si)[i]); tstride.push_back(shape::strideOf(si)[i]); }
      else { oshape.push_back(shape::shapeOf(si)[i]); ostride.push_back(shape::strideOf(si)[i]); }
    }
    auto tsi = makeShapeInfo(dt, shape::order(si), tshape, tstride.data());
    pack->tadShape = cachedShapeBuffer(tsi.data());
    LongType n = 1;
    for (auto s : oshape) n *= s;
    pack->offsets.resize(n);
    for (LongType t = 0; t < n; t++) {
      LongType idx = t, off = 0;
      for (int i = (int)oshape.size() - 1; i >= 0; i--) { off += (idx % oshape[i]) * ostride[i]; idx /= oshape[i]; }
      pack->offsets[t] = off;
    }
    pack->numTads = n;
  }
  auto* raw = pack.get();
  cache.emplace(std::make_pair(std::move(key), std::move(nd)), std::move(pack));
  return raw;
}

// ---- context --------------------------------------------------------------------------------------
NDArray* Context::input(int i) const {
  ND4J_REQUIRE(i >= 0 && i < (int)inputs.size() && inputs[i], "Context: input array " + std::to_string(i) + " is missing");
  return inputs[i];
}
NDArray* Context::output(int i) const {
  ND4J_REQUIRE(i >= 0 && i < (int)outputs.size() && outputs[i], "Context: output array " + std::to_string(i) + " is missing");
  return outputs[i];
}

}  // namespace nd4jhip
