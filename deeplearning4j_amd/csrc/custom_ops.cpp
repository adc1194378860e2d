// Declarable ops on the decoder path: matmul (+aliases), softmax, layer_norm, dot_product_attention_v2,
// argmax/argmin, and the glue ops a GPT-2-shaped decode step needs (gather, add, multiply, concat).
#include "custom_ops.h"

#include <algorithm>
#include <map>
#include <mutex>

#include "kernels.h"
#include "plan.h"

namespace nd4jhip {
namespace ops {

// ---- hash ----------------------------------------------------------------------------------------------------
LongType opHash(const std::string& name) {
  static unsigned long long table[256];
  static std::once_flag once;
  std::call_once(once, [] {
    unsigned long long h = 0x544B2FBACAAF1684ULL;
    for (int i = 0; i < 256; i++) {
      for (int j = 0; j < 31; j++) {
        h = (h >> 7) ^ h;
        h = (h << 11) ^ h;
        h = (h >> 10) ^ h;
      }
      table[i] = h;
    }
  });
  unsigned long long h = 0xBB40E64DA205B064ULL;
  const unsigned long long mult = 7664345821815920749ULL;
  for (char ch : name) {
    unsigned char uch = (unsigned char)ch;
    h = (h * mult) ^ table[uch & 0xff];
    h = (h * mult) ^ table[(uch >> 8) & 0xff];  // an 8-bit value shifted by 8: always entry 0, as in the reference
  }
  return (LongType)h;
}

static hipStream_t stream() { return LaunchContext::defaultContext()->execStream; }
static LongType iArg(const Context& c, size_t i, LongType def) { return i < c.iArgs.size() ? c.iArgs[i] : def; }
static double tArg(const Context& c, size_t i, double def) { return i < c.tArgs.size() ? c.tArgs[i] : def; }
static bool bArg(const Context& c, size_t i, bool def) { return i < c.bArgs.size() ? (bool)c.bArgs[i] : def; }
static std::vector<LongType> shapeOf(const NDArray* a) {
  return std::vector<LongType>(shape::shapeOf(a->shapeInfo()), shape::shapeOf(a->shapeInfo()) + a->rankOf());
}
static std::string shapeStr(const NDArray* a) {
  std::string s = "[";
  for (int i = 0; i < a->rankOf(); i++) s += (i ? "," : "") + std::to_string(a->sizeAt(i));
  return s + "]";
}

// ---- matmul ----------------------------------------------------------------------------------------------------
// generic/blas/matmul.cpp:35-176 of the reference: C = alpha * op(A) op(B) + beta * C; IArgs [transX, transY, transZ],
// TArgs [alpha, beta]; transZ swaps the inputs and flips both flags.  Transposes are realised through strides
// (the reference materialises permuted copies, helpers/impl/MmulHelper.cpp:506-526).
struct MatmulGeometry {
  NDArray *x, *y;
  bool transX, transY;
  LongType M, N, K;
  LongType aRow, aCol, bRow, bCol;
  std::vector<LongType> batchShape, xBatch, yBatch;
  std::vector<LongType> zShape;
};
static MatmulGeometry matmulGeometry(Context& c) {
  MatmulGeometry g;
  g.x = c.input(0); g.y = c.input(1);
  g.transX = iArg(c, 0, 0) != 0; g.transY = iArg(c, 1, 0) != 0;
  const bool transZ = iArg(c, 2, 0) != 0;
  if (transZ) {
    std::swap(g.x, g.y);
    bool t = g.transX; g.transX = !g.transY; g.transY = !t;
  }
  NDArray *x = g.x, *y = g.y;
  int xr = x->rankOf(), yr = y->rankOf();
  ND4J_REQUIRE(xr > 0 && yr > 0, "MATMUL OP: input arrays must have rank bigger than 0 (should not be scalars), but got instead: x rank = " + std::to_string(xr) + ", y rank = " + std::to_string(yr) + " !");
  // effective last-two dims and batch dims of x
  auto split = [](NDArray* a, bool trans, LongType& rows, LongType& cols, LongType& rs, LongType& cs, std::vector<LongType>& bshape, std::vector<LongType>& bstride, bool isX) {
    int r = a->rankOf();
    if (r == 1) {
      if (isX) { rows = 1; cols = a->sizeAt(0); rs = 0; cs = a->strideAt(0); }
      else { rows = a->sizeAt(0); cols = 1; rs = a->strideAt(0); cs = 0; }
      return;
    }
    int ri = trans ? r - 1 : r - 2, ci = trans ? r - 2 : r - 1;
    rows = a->sizeAt(ri); cols = a->sizeAt(ci); rs = a->strideAt(ri); cs = a->strideAt(ci);
    for (int d = 0; d < r - 2; d++) { bshape.push_back(a->sizeAt(d)); bstride.push_back(a->strideAt(d)); }
  };
  LongType Ky;
  std::vector<LongType> xbs, ybs;
  split(x, g.transX, g.M, g.K, g.aRow, g.aCol, xbs, g.xBatch, true);
  split(y, g.transY, Ky, g.N, g.bRow, g.bCol, ybs, g.yBatch, false);
  if (xr == 1 && yr == 1) {
    ND4J_REQUIRE(g.K == Ky, "MATMUL OP: since input arrays are vectors they must have the same length, but got x length = " + std::to_string(g.K) + ", y length = " + std::to_string(Ky) + " !");
    g.zShape = {};
  } else if (xr == 1 && yr == 2) {
    ND4J_REQUIRE(g.K == Ky, "MATMUL OP: input arrays have inconsistent shapes for vector-matrix product: x " + shapeStr(x) + ", y " + shapeStr(y) + " !");
    g.zShape = {g.N};
  } else if (xr == 2 && yr == 1) {
    ND4J_REQUIRE(g.K == Ky, "MATMUL OP: input arrays have inconsistent shapes for matrix-vector product: x " + shapeStr(x) + ", y " + shapeStr(y) + " !");
    g.zShape = {g.M};
  } else {
    // leading singleton dims of the higher-rank operand are squeezed against a rank-2 partner (matmul.cpp:80-118)
    auto allOnes = [](const std::vector<LongType>& v) { return std::all_of(v.begin(), v.end(), [](LongType s) { return s == 1; }); };
    if (xr != yr) {
      ND4J_REQUIRE((xr > yr && yr == 2 && allOnes(xbs)) || (yr > xr && xr == 2 && allOnes(ybs)),
                   "MATMUL OP: input and output arrays must have the same rank, but got instead: x rank = " + std::to_string(xr) + ", y rank = " + std::to_string(yr) + " !");
      g.zShape = xr > yr ? xbs : ybs;
      g.batchShape.clear(); g.xBatch.clear(); g.yBatch.clear();
    } else {
      for (size_t d = 0; d < xbs.size(); d++)
        ND4J_REQUIRE(xbs[d] == ybs[d], "MATMUL OP: input/output arrays have inconsistent shapes for matrix product: x " + shapeStr(x) + ", y " + shapeStr(y) + " !");
      g.batchShape = xbs;
      g.zShape = xbs;
    }
    ND4J_REQUIRE(g.K == Ky, "MATMUL OP: input/output arrays have inconsistent shapes for matrix product: x " + shapeStr(x) + ", y " + shapeStr(y) + " !");
    g.zShape.push_back(g.M); g.zShape.push_back(g.N);
  }
  return g;
}

static std::vector<std::vector<LongType>> matmulShapeFn(Context& c) {
  MatmulGeometry g = matmulGeometry(c);
  // order 'c' iff both inputs are 'c'; dtype = the higher of the two codes (matmul.cpp:189-219)
  char order = g.x->ordering() == 'c' && g.y->ordering() == 'c' ? 'c' : 'f';
  DataType dt = g.x->dataType() > g.y->dataType() ? g.x->dataType() : g.y->dataType();
  if (g.x->isEmpty() || g.y->isEmpty()) return {makeShapeInfo(g.x->dataType(), order, g.zShape, nullptr, ARRAY_EMPTY)};
  return {makeShapeInfo(dt, order, g.zShape)};
}

static void matmulExec(Context& c) {
  ND4J_REQUIRE(c.width() >= 2, "MATMUL OP: two input arrays are required");
  NDArray* z = c.output(0);
  if (c.input(0)->isEmpty() || c.input(1)->isEmpty()) return;
  MatmulGeometry g = matmulGeometry(c);
  ND4J_REQUIRE(z->lengthOf() == [&] { LongType n = 1; for (auto s : g.zShape) n *= s; return n; }(),
               "NDArrayFactory::matmul static method: input shape of output array is wrong, actual is " + shapeStr(z) + " !");
  // z must carry the expected shape up to unit dims
  {
    std::vector<LongType> a, b;
    for (auto s : g.zShape) if (s != 1) a.push_back(s);
    for (int d = 0; d < z->rankOf(); d++) if (z->sizeAt(d) != 1) b.push_back(z->sizeAt(d));
    ND4J_REQUIRE(a == b, "NDArrayFactory::matmul static method: input shape of output array is wrong, actual is " + shapeStr(z) + " !");
  }
  if (z->isEmpty()) return;
  DataType dt = z->dataType();
  ND4J_REQUIRE(g.x->dataType() == dt && g.y->dataType() == dt, "MATMUL OP: nd4j-hip requires x, y and z to share one data type");
  ND4J_REQUIRE(isFloatType(dt) || dt == INT32 || dt == INT64, std::string("MATMUL OP: ") + dtypeName(dt) + " arrays are not implemented in nd4j-hip");
  GemmDesc d;
  d.M = g.M; d.N = g.N; d.K = g.K;
  d.aRow = g.aRow; d.aCol = g.aCol; d.bRow = g.bRow; d.bCol = g.bCol;
  d.alpha = (float)tArg(c, 0, 1.0); d.beta = (float)tArg(c, 1, 0.0);
  // strides of z's matrix dims: the non-unit dims of z in order, lined up with [batch.., M, N]
  std::vector<LongType> zs;   // stride per entry of zShape
  {
    int zd = 0;
    for (size_t i = 0; i < g.zShape.size(); i++) {
      if (g.zShape[i] == 1) { zs.push_back(0); continue; }
      while (zd < z->rankOf() && z->sizeAt(zd) == 1) zd++;
      zs.push_back(z->strideAt(zd++));
    }
  }
  const int xr = g.x->rankOf(), yr = g.y->rankOf();
  if (xr == 1 && yr == 1) { d.cRow = 0; d.cCol = 0; }
  else if (xr == 1) { d.cRow = 0; d.cCol = zs.empty() ? 0 : zs.back(); }
  else if (yr == 1) { d.cRow = zs.empty() ? 0 : zs.back(); d.cCol = 0; }
  else { d.cRow = zs[zs.size() - 2]; d.cCol = zs[zs.size() - 1]; }
  // batch dims: collapse jointly; what does not collapse into one dim is looped on the host
  std::vector<LongType> bshape = g.batchShape, xb = g.xBatch, yb = g.yBatch, zb;
  for (size_t i = 0; i < bshape.size(); i++) zb.push_back(zs[i]);
  int br = 0;
  if (!bshape.empty()) {
    LongType* ptr[3] = {xb.data(), yb.data(), zb.data()};
    br = collapseDims((int)bshape.size(), bshape.data(), ptr, 3);
    bshape.resize(br); xb.resize(br); yb.resize(br); zb.resize(br);
    if (br == 1 && bshape[0] == 1) br = 0;
  }
  // with beta != 0 the output is read as well: its current contents must be on the device
  std::vector<NDArray*> reads = {g.x, g.y};
  if (d.beta != 0.f) reads.push_back(z);
  prepareSpecialUse(std::vector<NDArray*>{z}, reads);
  const size_t es = sizeOf(dt);
  const char* A = (const char*)g.x->specialBuffer();
  const char* B = (const char*)g.y->specialBuffer();
  char* C = (char*)z->specialBuffer();
  if (br == 0) {
    d.batch = 1;
    launchGemm(stream(), dt, A, B, C, d);
  } else {
    d.batch = bshape[br - 1]; d.aBatch = xb[br - 1]; d.bBatch = yb[br - 1]; d.cBatch = zb[br - 1];
    int inKernel = 1;   // batch dims resolved inside the kernel; the rest is looped here
    if (br >= 2 && bshape[br - 2] * bshape[br - 1] < 65536) {
      d.batchInner = bshape[br - 1]; d.batch = bshape[br - 2] * bshape[br - 1];
      d.aBatch2 = xb[br - 2]; d.bBatch2 = yb[br - 2]; d.cBatch2 = zb[br - 2];
      inKernel = 2;
    }
    LongType outer = 1;
    for (int i = 0; i < br - inKernel; i++) outer *= bshape[i];
    for (LongType o = 0; o < outer; o++) {
      LongType idx = o, ao = 0, bo = 0, co = 0;
      for (int i = br - inKernel - 1; i >= 0; i--) { LongType q = idx % bshape[i]; idx /= bshape[i]; ao += q * xb[i]; bo += q * yb[i]; co += q * zb[i]; }
      launchGemm(stream(), dt, A + ao * es, B + bo * es, C + co * es, d);
    }
  }
  registerSpecialUse(std::vector<NDArray*>{z}, reads);
}

// ---- xw_plus_b ---------------------------------------------------------------------------------------------------
// generic/nn/xw_plus_b.cpp:36-160: z = x w + b with b a row vector over the output features.  IArgs (each "== 1"):
// [transpose x, transpose w, transpose z]; x of rank > 2 is flattened to [prod(leading dims), last] (the reference
// reshapes it 'c', so it must be dense here).  The reference runs mmul and then addiRowVector; here the bias row is
// added in the product's epilogue (one rounding instead of two for 16-bit types).
struct XwGeometry {
  LongType M, N, K;
  LongType aRow, aCol, bRow, bCol, cRow, cCol;
  std::vector<LongType> zShape;
};
static bool denseC(const NDArray* a) {
  LongType expect = 1;
  for (int d = a->rankOf() - 1; d >= 0; d--) {
    if (a->sizeAt(d) != 1 && a->strideAt(d) != expect) return false;
    expect *= a->sizeAt(d);
  }
  return true;
}
static XwGeometry xwGeometry(Context& c, bool needOutput) {
  ND4J_REQUIRE(c.width() >= 3, "xw_plus_b: x, weights and bias are required");
  NDArray* x = c.input(0); NDArray* w = c.input(1); NDArray* b = c.input(2);
  const bool aT = iArg(c, 0, 0) == 1, bT = iArg(c, 1, 0) == 1, cT = iArg(c, 2, 0) == 1;
  XwGeometry g;
  std::vector<LongType> lead;
  ND4J_REQUIRE(x->rankOf() >= 2, "xw_plus_b: After reshaping, input x array should have rank equal 2, but got instead " + std::to_string(x->rankOf()) + "!");
  ND4J_REQUIRE(w->rankOf() == 2, "xw_plus_b: Input weights array should have rank equal 2, but got instead " + std::to_string(w->rankOf()) + "!");
  if (x->rankOf() > 2) {
    ND4J_REQUIRE(denseC(x), "xw_plus_b: nd4j-hip needs a dense c-order x of rank > 2 (it is flattened to two dims)");
    LongType m = 1;
    for (int d = 0; d < x->rankOf() - 1; d++) { m *= x->sizeAt(d); lead.push_back(x->sizeAt(d)); }
    g.M = m; g.K = x->sizeAt(x->rankOf() - 1); g.aRow = g.K; g.aCol = 1;
  } else {
    g.M = x->sizeAt(0); g.K = x->sizeAt(1); g.aRow = x->strideAt(0); g.aCol = x->strideAt(1);
    lead = {g.M};
  }
  if (aT) { std::swap(g.M, g.K); std::swap(g.aRow, g.aCol); lead = {g.M}; }
  LongType Kw = w->sizeAt(0);
  g.N = w->sizeAt(1); g.bRow = w->strideAt(0); g.bCol = w->strideAt(1);
  if (bT) { std::swap(Kw, g.N); std::swap(g.bRow, g.bCol); }
  ND4J_REQUIRE(Kw == g.K, "xw_plus_b: input arrays have inconsistent shapes for matrix product: x " + shapeStr(x) + ", weights " + shapeStr(w) + " !");
  ND4J_REQUIRE(b->lengthOf() == g.N, "xw_plus_b: Input bias vector should be 1D and have proper dimension 1x" + std::to_string(g.N) + ". But got length " + std::to_string(b->lengthOf()) + " instead !");
  g.zShape = lead; g.zShape.push_back(g.N);
  if (cT) { ND4J_REQUIRE(g.zShape.size() == 2, "xw_plus_b: a transposed output needs a rank-2 product"); std::swap(g.zShape[0], g.zShape[1]); }
  if (needOutput) {
    NDArray* z = c.output(0);
    ND4J_REQUIRE(shapeOf(z) == g.zShape, "xw_plus_b: output array has shape " + shapeStr(z) + ", expected the product's shape");
    if (z->rankOf() > 2) {
      ND4J_REQUIRE(denseC(z), "xw_plus_b: nd4j-hip needs a dense c-order output of rank > 2");
      g.cRow = g.N; g.cCol = 1;
    } else {
      g.cRow = z->strideAt(0); g.cCol = z->strideAt(1);
      if (cT) std::swap(g.cRow, g.cCol);
    }
  }
  return g;
}
// epi: extra outputs for the product's epilogue (already prepared for device use by the caller); returns whether the kernel
// that ran wrote them
// out = layer_norm(x; gain, bias) is the product's input: `rows` rows of unit element stride, xPitch / outPitch elements apart
struct LnPrologue { NDArray *x, *gain, *bias, *out; LongType rows, xPitch, outPitch; };
// the product's input row is the output of an attention that left the records of its key ranges in `partial` (device memory):
// the product merges them on its way in and writes the row to `out` as well
struct AttnMergePrologue { const float* partial; int splits, D; NDArray* out; };
static bool xwPlusBImpl(Context& c, const GemmEpilogue* epi, const LnPrologue* ln = nullptr, const AttnMergePrologue* am = nullptr) {
  ND4J_REQUIRE(c.width() >= 3, "xw_plus_b: x, weights and bias are required");
  NDArray* x = c.input(0); NDArray* w = c.input(1); NDArray* b = c.input(2); NDArray* z = c.output(0);
  if (x->isEmpty() || w->isEmpty() || b->isEmpty()) return epi == nullptr;
  XwGeometry g = xwGeometry(c, true);
  const DataType dt = z->dataType();
  ND4J_REQUIRE(x->dataType() == dt && w->dataType() == dt && b->dataType() == dt && isFloatType(dt), "xw_plus_b: nd4j-hip requires one floating point type for x, weights, bias and output");
  // the bias row is read as a dense vector
  LongType bstride = 1;
  for (int d = 0; d < b->rankOf(); d++) if (b->sizeAt(d) != 1) bstride = b->strideAt(d);
  ND4J_REQUIRE(bstride == 1 || g.N == 1, "xw_plus_b: nd4j-hip needs a contiguous bias vector");
  GemmDesc d;
  d.M = g.M; d.N = g.N; d.K = g.K;
  d.aRow = g.aRow; d.aCol = g.aCol; d.bRow = g.bRow; d.bCol = g.bCol; d.cRow = g.cRow; d.cCol = g.cCol;
  if (ln) {
    // the product reads the row before normalisation and writes the normalised row where the separate op would have
    if (g.M != ln->rows || g.aCol != 1 || ln->x->lengthOf() != g.M * g.K || ln->x->dataType() != dt) return false;
    prepareSpecialUse({z, ln->out}, {ln->x, ln->gain, ln->bias, w, b});
    d.bias = b->specialBuffer();
    d.epi = epi;
    d.aRow = ln->xPitch;
    d.lnGain = ln->gain->specialBuffer(); d.lnBias = ln->bias->specialBuffer(); d.lnOut = ln->out->specialBuffer(); d.lnOutRow = ln->outPitch;
    const bool done = launchGemm(stream(), dt, ln->x->specialBuffer(), w->specialBuffer(), z->specialBuffer(), d);
    if (done) registerSpecialUse({z, ln->out}, {ln->x, ln->gain, ln->bias, w, b});
    return done;
  }
  if (am) {
    if (g.M != 1 || g.aCol != 1 || am->out->lengthOf() != g.K || am->out->dataType() != dt) return false;
    prepareSpecialUse({z, am->out}, {w, b});
    d.bias = b->specialBuffer();
    d.epi = epi;
    d.attnPartial = am->partial; d.attnSplits = am->splits; d.attnD = am->D; d.attnOut = am->out->specialBuffer();
    const bool done = launchGemm(stream(), dt, am->out->specialBuffer(), w->specialBuffer(), z->specialBuffer(), d);
    if (done) registerSpecialUse({z, am->out}, {w, b});
    return done;
  }
  prepareSpecialUse({z}, {x, w, b});
  d.bias = b->specialBuffer();
  d.epi = epi;
  const bool applied = launchGemm(stream(), dt, x->specialBuffer(), w->specialBuffer(), z->specialBuffer(), d);
  registerSpecialUse({z}, {x, w, b});
  return applied;
}
static void xwPlusBExec(Context& c) { xwPlusBImpl(c, nullptr); }
static std::vector<std::vector<LongType>> xwPlusBShapeFn(Context& c) {
  XwGeometry g = xwGeometry(c, false);
  return {makeShapeInfo(c.input(0)->dataType(), 'c', g.zShape)};
}

// ---- softmax -----------------------------------------------------------------------------------------------------
// generic/nn/softmax.cpp:37-52 -> helpers/cpu/softmax.cpp:252-353
static bool sameShapeStrict(const NDArray* a, const NDArray* b) {
  if (a->rankOf() != b->rankOf()) return false;
  for (int d = 0; d < a->rankOf(); d++) if (a->sizeAt(d) != b->sizeAt(d) || a->strideAt(d) != b->strideAt(d)) return false;
  return true;
}
static bool isVector(const NDArray* a) {
  if (a->rankOf() == 1) return true;
  if (a->rankOf() == 2) return (a->sizeAt(0) == 1 || a->sizeAt(1) == 1) && a->lengthOf() > 1;
  return false;
}
static void fillValue(NDArray* z, double v) {
  EwPlan p = buildEwPlan({z->shapeInfo(), z->shapeInfo()});
  launchScalarOp(stream(), P_COPY, z->dataType(), z->specialBuffer(), v, z->specialBuffer(), p);
}
static void softmaxExec(Context& c) {
  NDArray* x = c.input(0);
  NDArray* z = c.output(0);
  const int rank = x->rankOf();
  int dim = (int)iArg(c, 0, rank - 1);
  ND4J_REQUIRE(dim < rank, "SOFTMAX OP: the value of input integer parameter (dimension) must be less than input array rank " + std::to_string(rank) + ", but got dimension = " + std::to_string(dim) + " instead !");
  if (dim < 0) dim += rank;
  ND4J_REQUIRE(rank == 0 || dim >= 0, "SOFTMAX OP: dimension out of range");
  ND4J_REQUIRE(x->dataType() == z->dataType() && isFloatType(x->dataType()), "SOFTMAX OP: input and output must share a floating point type");
  ND4J_REQUIRE(x->lengthOf() == z->lengthOf(), "SOFTMAX OP: input and output lengths differ");
  if (x->isEmpty()) return;
  prepareSpecialUse({z}, {x});
  bool clamp = sameShapeStrict(x, z);
  if (isVector(x)) {
    if (rank != 1 && x->sizeAt(dim) == 1) {  // softmax.cpp:255-259: a vector reduced along its unit axis is all ones
      fillValue(z, 1.0);
      registerSpecialUse({z}, {x});
      return;
    }
    // the vector path ignores `dim` and normalises the whole vector, always with the clamp semantics
    clamp = true;
    if (rank == 2) dim = x->sizeAt(0) == 1 ? 1 : 0;
  }
  if (rank == 0) { fillValue(z, 1.0); registerSpecialUse({z}, {x}); return; }
  RowPlan p = buildRowPlan(x->shapeInfo(), z->shapeInfo(), dim);
  launchSoftmax(stream(), x->dataType(), x->specialBuffer(), z->specialBuffer(), p, clamp);
  registerSpecialUse({z}, {x});
}
static std::vector<std::vector<LongType>> sameAsInputShapeFn(Context& c) {
  NDArray* x = c.input(0);
  return {makeShapeInfo(x->dataType(), x->ordering(), shapeOf(x))};
}

// log_softmax (generic/nn/logSoftmax.cpp:34-49): IArg0 = dim (default last); a vector is normalised whole unless dim names
// its unit axis, which gives zeros (helpers/cpu/activations.cpp:236-246)
static void logSoftmaxExec(Context& c) {
  NDArray* x = c.input(0);
  NDArray* z = c.output(0);
  const int rank = x->rankOf();
  int dim = (int)iArg(c, 0, rank - 1);
  ND4J_REQUIRE(dim < rank || rank == 0, "LOG_SOFTMAX OP: the value of input integer parameter (dimension) must be less than input array rank " + std::to_string(rank) + ", but got dimension = " + std::to_string(dim) + " instead !");
  if (dim < 0) dim += rank;
  ND4J_REQUIRE(rank == 0 || dim >= 0, "LOG_SOFTMAX OP: dimension out of range");
  ND4J_REQUIRE(x->dataType() == z->dataType() && isFloatType(x->dataType()), "LOG_SOFTMAX OP: input and output must share a floating point type");
  ND4J_REQUIRE(x->lengthOf() == z->lengthOf(), "LOG_SOFTMAX OP: input and output lengths differ");
  if (x->isEmpty()) return;
  prepareSpecialUse({z}, {x});
  if (rank == 0 || (isVector(x) && rank != 1 && x->sizeAt(dim) == 1)) {
    fillValue(z, 0.0);
  } else {
    if (isVector(x) && rank == 2) dim = x->sizeAt(0) == 1 ? 1 : 0;
    RowPlan p = buildRowPlan(x->shapeInfo(), z->shapeInfo(), dim);
    launchLogSoftmax(stream(), x->dataType(), x->specialBuffer(), z->specialBuffer(), p);
  }
  registerSpecialUse({z}, {x});
}

// statistics groups of a standardisation over `axes`: the reduced dims form the inner walk, the others the outer one;
// dimC (or -1) is the axis gain and bias run along
static LnGenericPlan lnGenericPlan(const NDArray* x, const NDArray* z, const std::vector<LongType>& axes, int dimC) {
  const int rank = x->rankOf();
  LnGenericPlan p;
  std::vector<bool> red(rank, false);
  for (auto a : axes) red[a] = true;
  std::vector<LongType> os, oxs, ozs, is, ixs, izs;
  for (int d = 0; d < rank; d++) {
    if (red[d]) { if (d == dimC) { p.channelInInner = 1; p.channelPos = (int)is.size(); } is.push_back(x->sizeAt(d)); ixs.push_back(x->strideAt(d)); izs.push_back(z->strideAt(d)); }
    else { if (d == dimC) { p.channelInInner = 0; p.channelPos = (int)os.size(); } os.push_back(x->sizeAt(d)); oxs.push_back(x->strideAt(d)); ozs.push_back(z->strideAt(d)); }
  }
  p.outerLen = 1; for (auto s : os) p.outerLen *= s;
  p.innerLen = 1; for (auto s : is) p.innerLen *= s;
  p.outerX = toDevShape(os, oxs); p.outerZ = toDevShape(os, ozs);
  p.innerX = toDevShape(is, ixs); p.innerZ = toDevShape(is, izs);
  return p;
}
// ---- layer_norm ------------------------------------------------------------------------------------------------------
// generic/nn/layer_norm.cpp:35-79: standardize over IArgs axes, then * gain (+ bias) along dim 1 (BArg0 true or
// absent) or the last dim (BArg0 false); eps 1e-5 inside the sqrt (generic/transforms/standardize.cpp:34-78)
static void layerNormImpl(Context& c, NDArray* x, NDArray* gain, NDArray* bias, NDArray* z, const std::vector<LongType>& axesIn, bool channelsFirst, const char* opName) {
  const int rank = x->rankOf();
  ND4J_REQUIRE(!axesIn.empty(), "STANDARDIZE OP: axis has to be non-empty");
  auto axes = normalizeDims(rank, axesIn.data(), (LongType)axesIn.size(), opName);
  ND4J_REQUIRE(x->dataType() == z->dataType() && isFloatType(x->dataType()), std::string(opName) + ": input and output must share a floating point type");
  ND4J_REQUIRE(sameShapeStrict(x, z) || shapeOf(x) == shapeOf(z), std::string(opName) + ": input and output shapes differ");
  int dimC = -1;
  if (gain) {
    dimC = channelsFirst ? 1 : rank - 1;
    ND4J_REQUIRE(dimC < rank, std::string(opName) + ": input rank too small for the channel axis");
    ND4J_REQUIRE(gain->rankOf() == 1 && gain->sizeAt(0) == x->sizeAt(dimC),
                 "LAYER_NORM OP: wrong shape of gain array, expected is {" + std::to_string(x->sizeAt(dimC)) + "}, but got " + shapeStr(gain) + " instead !");
    if (bias) ND4J_REQUIRE(bias->rankOf() == 1 && bias->sizeAt(0) == x->sizeAt(dimC),
                           "LAYER_NORM OP: wrong shape of bias array, expected is {" + std::to_string(x->sizeAt(dimC)) + "}, but got " + shapeStr(bias) + " instead !");
    ND4J_REQUIRE(gain->dataType() == x->dataType() && (!bias || bias->dataType() == x->dataType()), "LAYER_NORM OP: nd4j-hip requires gain and bias to carry the input's data type");
  }
  if (x->isEmpty()) return;
  std::vector<NDArray*> reads = {x};
  if (gain) reads.push_back(gain);
  if (bias) reads.push_back(bias);
  prepareSpecialUse(std::vector<NDArray*>{z}, reads);
  const float eps = 1e-5f;
  const bool lastAxisOnly = axes.size() == 1 && axes[0] == rank - 1 && dimC == rank - 1 && gain && gain->strideAt(0) == 1 && (!bias || bias->strideAt(0) == 1);
  bool done = false;
  if (lastAxisOnly) {   // the row kernels say themselves which rows they take
    RowPlan p = buildRowPlan(x->shapeInfo(), z->shapeInfo(), rank - 1);
    done = launchLayerNormRows(stream(), x->dataType(), x->specialBuffer(), gain->specialBuffer(), bias ? bias->specialBuffer() : nullptr, z->specialBuffer(), p, eps);
  }
  if (!done) {
    ND4J_REQUIRE(!gain || (gain->strideAt(0) == 1 && (!bias || bias->strideAt(0) == 1)), "LAYER_NORM OP: gain/bias must be dense");
    LnGenericPlan p = lnGenericPlan(x, z, axes, dimC);
    launchLayerNormGeneric(stream(), x->dataType(), x->specialBuffer(), gain ? gain->specialBuffer() : nullptr, bias ? bias->specialBuffer() : nullptr, z->specialBuffer(), p, eps);
  }
  registerSpecialUse(std::vector<NDArray*>{z}, reads);
}
static void layerNormExec(Context& c) {
  ND4J_REQUIRE(c.width() >= 2, "LAYER_NORM OP: input and gain arrays are required");
  NDArray* bias = c.width() > 2 ? c.input(2) : nullptr;
  layerNormImpl(c, c.input(0), c.input(1), bias, c.output(0), c.iArgs, bArg(c, 0, true), "LAYER_NORM OP");
}

// ---- dot_product_attention_v2 ---------------------------------------------------------------------------------------------
// generic/nn/dot_product_attention_v2.cpp:35-125 -> helpers/impl/AttentionHelper.cpp:411-469.
// Inputs (queries, values, keys?); TArgs [scale, dropout]; BArgs [useCausalMask, training];
// Inputs 3 / 4: optional query mask [batch.., Tq] and value mask [batch.., Tv].
// outputs [out, weights?, logits?].  logits = clip(scale * q k^T, +-1e4) (scale applied unless 0 or 1),
// logits where the causal mask (j > i) or the value mask (cast to BOOL, false = padded key) hides the key get
// 65504 (bf16) / 1e9 (other types) subtracted once, weights = softmax(logits), out = weights v, and last the weights
// output is multiplied by the query mask (out is not: the reference forms it before).
// With only `out` supplied the fused kernel runs and nothing of size Tq x Tv is written.
// An operand seen as [outer, H, T, D]: rank 2 has no batch, rank 3 one batch level (H = 0), rank >= 4 two levels
// (the last leading dim is the inner level; the dims before it must fold into one).  The two-level form is what a
// [batch, heads, T, D] view of a token-major [batch, T, heads * D] buffer needs: its batch dims do not nest.
struct BatchedView {
  LongType B = 1, H = 0, T = 0, D = 0;     // B counts all batch entries
  LongType sB = 0, sB2 = 0, sT = 0, sD = 0;
};
static BatchedView batchedView(const NDArray* a, const char* what) {
  BatchedView r;
  const int rank = a->rankOf();
  ND4J_REQUIRE(rank >= 2, std::string("dot_product_attention_v2: ") + what + " must have rank >= 2");
  r.T = a->sizeAt(rank - 2); r.D = a->sizeAt(rank - 1); r.sT = a->strideAt(rank - 2); r.sD = a->strideAt(rank - 1);
  if (rank == 2) { r.B = 1; return r; }
  if (rank == 3) { r.B = a->sizeAt(0); r.sB = a->strideAt(0); return r; }
  std::vector<LongType> bs, bst;
  for (int d = 0; d < rank - 3; d++) { bs.push_back(a->sizeAt(d)); bst.push_back(a->strideAt(d)); }
  LongType* ptr[1] = {bst.data()};
  const int nr = collapseDims((int)bs.size(), bs.data(), ptr, 1);
  ND4J_REQUIRE(nr == 1, std::string("dot_product_attention_v2: leading dims of ") + what + " (rank " + std::to_string(rank) + ") do not fold into [batch, heads]");
  r.H = a->sizeAt(rank - 3); r.sB = a->strideAt(rank - 3);
  r.B = bs[0] * r.H; r.sB2 = bs[0] > 1 ? bst[0] : 0;   // a unit outer dim never moves
  return r;
}
static bool denseRows(const BatchedView& v) {   // row-major [B, T, D] without gaps
  if (v.sD != 1 || v.sT != v.D) return false;
  if (v.H > 0) return v.sB == v.T * v.D && v.sB2 == v.H * v.T * v.D;
  return v.B == 1 || v.sB == v.T * v.D;
}
// Set by a merged step of a recording around its call of the attention op: when the decode kernel cuts the key range up, it
// leaves the merge of the parts to the caller's next kernel and says here where the parts are.
struct AttnMergeRequest { bool deferred = false; AttnDesc desc; DataType dt = FLOAT32; };
static AttnMergeRequest* g_attnMergeRequest = nullptr;
static void attentionExec(Context& c) {
  ND4J_REQUIRE(c.width() >= 2, "dot_product_attention_v2: queries and values are required");
  NDArray* q0 = c.input(0); NDArray* v0 = c.input(1); NDArray* k0 = c.width() > 2 ? c.input(2) : v0;
  NDArray* o0 = c.output(0);
  ND4J_REQUIRE(q0->rankOf() == v0->rankOf(), "Queries and values must be same ranks!");
  // optional masks (dot_product_attention_v2.cpp:57-58): input 3 = query mask [batch.., Tq], input 4 = value mask [batch.., Tv]
  NDArray* qMask = c.width() > 3 && c.inputs[3] != nullptr && !c.inputs[3]->isEmpty() ? c.inputs[3] : nullptr;
  NDArray* vMask = c.width() > 4 && c.inputs[4] != nullptr && !c.inputs[4]->isEmpty() ? c.inputs[4] : nullptr;
  const double dropout = tArg(c, 1, 0.0);
  const double scale = tArg(c, 0, 1.0);
  const bool causal = bArg(c, 0, false), training = bArg(c, 1, false);
  ND4J_REQUIRE(!(training && dropout > 0.0), "dot_product_attention_v2: dropout is not implemented in nd4j-hip");
  const BatchedView q = batchedView(q0, "queries"), v = batchedView(v0, "values"), k = batchedView(k0, "keys"), out = batchedView(o0, "output");
  const bool wantW = c.outputs.size() > 1 && c.outputs[1] != nullptr, wantL = c.outputs.size() > 2 && c.outputs[2] != nullptr;
  DataType dt = q0->dataType();
  ND4J_REQUIRE(isFloatType(dt) && dt != DOUBLE, "dot_product_attention_v2: nd4j-hip implements FLOAT, HALF and BFLOAT16");
  ND4J_REQUIRE(k0->dataType() == dt && v0->dataType() == dt && o0->dataType() == dt, "dot_product_attention_v2: all arrays must share one data type");
  AttnDesc d;
  d.B = q.B; d.H = q.H; d.Tq = q.T; d.D = q.D; d.Tv = v.T; d.Dv = v.D;
  ND4J_REQUIRE(k.B == d.B && v.B == d.B && k.H == d.H && v.H == d.H, "dot_product_attention_v2: batch sizes differ");
  ND4J_REQUIRE(k.T == d.Tv && k.D == d.D, "dot_product_attention_v2: keys must be [batch, Tv, dim], got " + shapeStr(k0));
  ND4J_REQUIRE(out.B == d.B && out.H == d.H && out.T == d.Tq && out.D == d.Dv, "dot_product_attention_v2: output must be [batch, Tq, dimV], got " + shapeStr(o0));
  d.scale = (float)scale; d.applyScale = scale != 0.0 && scale != 1.0; d.causal = causal;
  d.maskValue = dt == BFLOAT16 ? 65504.0f : 1.0e9f;
  std::vector<NDArray*> reads = {q0, v0, k0};
  std::vector<NDArray*> writes = {o0};
  if (wantW) writes.push_back(c.outputs[1]);
  if (wantL) writes.push_back(c.outputs[2]);
  // a mask carries the batch dims of the queries followed by the sequence length (the reference expands it at -2 / -1
  // and lets it broadcast against [batch.., Tq, Tv], AttentionHelper.cpp:434-436,463-466)
  auto maskFits = [&](NDArray* m, LongType T, const char* what) {
    bool ok = m->rankOf() == std::max(q0->rankOf() - 1, 1) && m->lengthOf() == d.B * T && m->sizeAt(-1) == T;
    for (int i = 0; ok && i < m->rankOf() - 1; i++) ok = m->sizeAt(i) == q0->sizeAt(i);
    ND4J_REQUIRE(ok, std::string("dot_product_attention_v2: the ") + what + " mask must have shape [batch.., " + std::to_string(T) + "], got " + shapeStr(m));
    ND4J_REQUIRE(isFloatType(m->dataType()) || m->dataType() == BOOL || m->dataType() == INT32 || m->dataType() == INT64,
                 std::string("dot_product_attention_v2: unsupported data type of the ") + what + " mask");
  };
  if (vMask) { maskFits(vMask, d.Tv, "value"); reads.push_back(vMask); }
  if (qMask) { maskFits(qMask, d.Tq, "query"); reads.push_back(qMask); }
  if (d.B * d.Tq == 0) return;
  prepareSpecialUse(writes, reads);
  d.qB = q.sB; d.qT = q.sT; d.kB = k.sB; d.kT = k.sT; d.vB = v.sB; d.vT = v.sT; d.oB = out.sB; d.oT = out.sT;
  d.qB2 = q.sB2; d.kB2 = k.sB2; d.vB2 = v.sB2; d.oB2 = out.sB2;
  const bool unitInner = q.sD == 1 && k.sD == 1 && v.sD == 1 && out.sD == 1;
  const bool useDecode = !wantW && !wantL && unitInner && attentionDecodeSupported(dt, d);
  // (the fp32 tile kernel takes no value mask; d.vmask is only filled in below)
  const bool useFused = !useDecode && !wantW && !wantL && unitInner && !(dt == FLOAT32 && vMask) && attentionFusedSupported(dt, d);
  // Temporaries (dense copies of the masks; logits and weights of the composition when they are not outputs) are carved out
  // of the launch context's grow-only scratch: no allocation and no wait per call once it has grown to the problem's size.
  const LongType lw = d.Tq * d.Tv;
  auto round256 = [](size_t b) { return (b + 255) & ~(size_t)255; };
  size_t need = 0;
  if (vMask) need += round256((size_t)vMask->lengthOf());
  if (qMask && wantW) need += round256((size_t)qMask->lengthOf() * sizeOf(dt));
  if (!useDecode && !useFused) need += (wantL ? 0 : round256((size_t)(d.B * lw) * sizeOf(dt))) + (wantW ? 0 : round256((size_t)(d.B * lw) * sizeOf(dt)));
  char* ws = need ? static_cast<char*>(LaunchContext::defaultContext()->workspace(need)) : nullptr;
  auto carve = [&](size_t bytes) { char* p = ws; ws += round256(bytes); return static_cast<void*>(p); };
  // dense device copies of the masks in the form the kernels read: the value mask as bytes (cast to BOOL: non-zero keeps
  // the key), the query mask in the arrays' type.  A mask that already is dense and of that type is used in place.
  auto denseMask = [&](NDArray* m, DataType want) -> const void* {
    auto dsi = makeShapeInfo(want, 'c', shapeOf(m));
    void* copy = carve((size_t)m->lengthOf() * sizeOf(want));   // (carved either way: the sum above counted it)
    if (m->dataType() == want) {
      bool dense = true;
      for (int i = 0; i < m->rankOf(); i++) if (m->sizeAt(i) != 1 && m->strideAt(i) != shape::strideOf(dsi.data())[i]) dense = false;
      if (dense) return m->specialBuffer();
    }
    EwPlan p = buildEwPlan({dsi.data(), m->shapeInfo()});
    launchUnary(stream(), U_IDENTITY, m->dataType(), want, m->specialBuffer(), copy, p);
    return copy;
  };
  if (vMask) d.vmask = static_cast<const unsigned char*>(denseMask(vMask, BOOL));
  // the query mask scales the weights output only: out = weights v has been formed before (AttentionHelper.cpp:455-467)
  const void* qm = qMask && wantW ? denseMask(qMask, dt) : nullptr;
  if (useDecode) {
    const int cut = attentionDecodeSplits(d);
    if (cut > 1 && (size_t)(d.B * d.Tq * cut) * (size_t)(d.D + 4) * sizeof(float) <= LaunchContext::ALLOCATION_BYTES) {
      // the parts' records go to the scratch the split-K products use: written and read back by kernels that follow each other
      d.splits = cut;
      d.partial = static_cast<float*>(LaunchContext::defaultContext()->allocationBuffer);
      if (g_attnMergeRequest != nullptr) { d.mergeLater = true; g_attnMergeRequest->deferred = true; g_attnMergeRequest->desc = d; g_attnMergeRequest->dt = dt; }
    }
    launchAttentionDecode(stream(), dt, q0->specialBuffer(), k0->specialBuffer(), v0->specialBuffer(), o0->specialBuffer(), d);
  } else if (useFused) {
    launchAttentionFused(stream(), dt, q0->specialBuffer(), k0->specialBuffer(), v0->specialBuffer(), o0->specialBuffer(), d);
  } else {
    // composition: logits = q k^T -> fix-up (scale, clip, mask) -> softmax -> out = weights v
    auto denseOutput = [&](NDArray* a, const char* what) {
      const BatchedView b = batchedView(a, what);
      ND4J_REQUIRE(b.B == d.B && b.T == d.Tq && b.D == d.Tv && a->dataType() == dt && denseRows(b),
                   std::string("dot_product_attention_v2: ") + what + " output must be a dense row-major [batch, Tq, Tv] array");
      return a->specialBuffer();
    };
    void* logits = wantL ? denseOutput(c.outputs[2], "logits") : carve((size_t)(d.B * lw) * sizeOf(dt));
    void* weights = wantW ? denseOutput(c.outputs[1], "weights") : carve((size_t)(d.B * lw) * sizeOf(dt));
    GemmDesc g1;
    g1.M = d.Tq; g1.N = d.Tv; g1.K = d.D; g1.batch = d.B; g1.batchInner = d.H;
    g1.aRow = q.sT; g1.aCol = q.sD; g1.aBatch = q.sB; g1.aBatch2 = q.sB2;
    g1.bRow = k.sD; g1.bCol = k.sT; g1.bBatch = k.sB; g1.bBatch2 = k.sB2;   // k^T
    g1.cRow = d.Tv; g1.cCol = 1; g1.cBatch = lw; g1.cBatch2 = d.H * lw;
    launchGemm(stream(), dt, q0->specialBuffer(), k0->specialBuffer(), logits, g1);
    launchAttentionLogitsFixup(stream(), dt, logits, d);
    auto si3 = makeShapeInfo(dt, 'c', {d.B, d.Tq, d.Tv});
    RowPlan rp = buildRowPlan(si3.data(), si3.data(), 2);
    launchSoftmax(stream(), dt, logits, weights, rp, true);
    GemmDesc g2;
    g2.M = d.Tq; g2.N = d.Dv; g2.K = d.Tv; g2.batch = d.B; g2.batchInner = d.H;
    g2.aRow = d.Tv; g2.aCol = 1; g2.aBatch = lw; g2.aBatch2 = d.H * lw;
    g2.bRow = v.sT; g2.bCol = v.sD; g2.bBatch = v.sB; g2.bBatch2 = v.sB2;
    g2.cRow = out.sT; g2.cCol = out.sD; g2.cBatch = out.sB; g2.cBatch2 = out.sB2;
    launchGemm(stream(), dt, weights, v0->specialBuffer(), o0->specialBuffer(), g2);
    if (qm) launchAttentionQueryMask(stream(), dt, weights, qm, d);
  }
  registerSpecialUse(writes, reads);
}
static std::vector<std::vector<LongType>> attentionShapeFn(Context& c) {
  // The reference's shape function (dot_product_attention_v2.cpp:132-183) reports [batch, Tq, dim] for the weights
  // and logits of rank-3 inputs, which cannot hold what doAttention writes; this one reports [batch, Tq, Tv].
  NDArray* q = c.input(0); NDArray* v = c.input(1);
  DataType dt = q->dataType();
  std::vector<LongType> qs = shapeOf(q), vs = shapeOf(v);
  ND4J_REQUIRE(qs.size() >= 2 && qs.size() == vs.size(), "Queries and values must be same ranks!");
  std::vector<LongType> o(qs.begin(), qs.end() - 1), w(qs.begin(), qs.end() - 1);
  o.push_back(vs.back());
  w.push_back(vs[vs.size() - 2]);
  return {makeShapeInfo(dt, 'c', o), makeShapeInfo(dt, 'c', w), makeShapeInfo(dt, 'c', w)};
}

// ---- top_k -----------------------------------------------------------------------------------------------------------------
// generic/parity_ops/top_k.cpp:31-57: k from IArg0 or from a second input; BArg0 = sort by value (default true, else the
// picks come in index order); outputs [values (input type), indices (INT64 by the shape function)] with the last
// dim replaced by k.  For k = 1 the first maximum wins, as in the reference.  For k > 1 the reference's insertion
// loop (helpers/cpu/top_k.cpp:62-99) never admits a value that is already in its candidate set and recovers
// positions by value afterwards, so rows with repeated values among the winners give it fewer distinct picks or one
// position twice; this implementation returns the k largest elements with ties resolved to the lower index, which
// is the same result whenever the winners are pairwise different.
static int topKCount(Context& c) {
  if (c.width() > 1) {
    NDArray* ka = c.input(1);
    ka->buf->syncToPrimary();
    ND4J_REQUIRE(ka->lengthOf() >= 1, "top_k: k array is empty");
    if (ka->dataType() == INT64) return (int)ka->hostAs<LongType>()[0];
    if (ka->dataType() == INT32) return ka->hostAs<int>()[0];
    ND4J_THROW("top_k: k array must be INT32 or INT64");
  }
  return (int)iArg(c, 0, 1);
}
static std::vector<LongType> widened(const NDArray* z, LongType n) {
  // z's descriptor with the last extent set to n: lets the row planner pair it with x
  std::vector<LongType> shp = shapeOf(z), st;
  for (int d = 0; d < z->rankOf(); d++) st.push_back(z->strideAt(d));
  shp.back() = n;
  return makeShapeInfo(z->dataType(), 'c', shp, st.data());
}
static void topKExec(Context& c) {
  NDArray* x = c.input(0);
  ND4J_REQUIRE(c.outputs.size() >= 2 && c.outputs[0] && c.outputs[1], "top_k: values and indices outputs are required");
  NDArray* v = c.output(0); NDArray* idx = c.outputs[1];
  const int k = topKCount(c);
  const bool needSort = bArg(c, 0, true);
  ND4J_REQUIRE(x->rankOf() >= 1, "top_k: input must have rank >= 1");
  const LongType n = x->sizeAt(x->rankOf() - 1);
  ND4J_REQUIRE(k <= n, "top_k: k should not be greater than last dimension");
  ND4J_REQUIRE(k > 0, "top_k: k should be positive, but " + std::to_string(k) + " given.");
  std::vector<LongType> want = shapeOf(x);
  want.back() = k;
  ND4J_REQUIRE(shapeOf(v) == want && shapeOf(idx) == want, "top_k: outputs must have the input's shape with the last dim replaced by k");
  ND4J_REQUIRE(v->dataType() == x->dataType(), "top_k: values must carry the input's data type");
  if (x->isEmpty()) return;
  auto vsi = widened(v, n), isi = widened(idx, n);
  RowPlan pv = buildRowPlan(x->shapeInfo(), vsi.data(), x->rankOf() - 1), pi = buildRowPlan(x->shapeInfo(), isi.data(), x->rankOf() - 1);
  prepareSpecialUse({v, idx}, {x});
  launchTopK(stream(), x->dataType(), idx->dataType(), x->specialBuffer(), v->specialBuffer(), idx->specialBuffer(), pv, pi, k, needSort);
  registerSpecialUse({v, idx}, {x});
}
static std::vector<std::vector<LongType>> topKShapeFn(Context& c) {
  NDArray* x = c.input(0);
  const int k = topKCount(c);
  ND4J_REQUIRE(k > 0, "top_k: k should be positive, but " + std::to_string(k) + " given.");
  std::vector<LongType> shp = shapeOf(x);
  ND4J_REQUIRE(!shp.empty(), "top_k: input must have rank >= 1");
  shp.back() = k;
  return {makeShapeInfo(x->dataType(), x->ordering(), shp), makeShapeInfo(INT64, x->ordering(), shp)};
}

// ---- argmax / argmin ---------------------------------------------------------------------------------------------------------
// generic/reduce/argmax.cpp:38-103: dims from IArgs or from input 1; BArg0 keepDims; DArg0 output dtype (INT64)
static std::vector<LongType> argDims(Context& c) {
  std::vector<LongType> dims = c.iArgs;
  if (c.width() > 1 && dims.empty()) {
    NDArray* ax = c.input(1);
    ax->buf->syncToPrimary();
    for (LongType i = 0; i < ax->lengthOf(); i++) {
      if (ax->dataType() == INT64) dims.push_back(ax->hostAs<LongType>()[i * (ax->rankOf() ? ax->strideAt(ax->rankOf() - 1) : 1)]);
      else if (ax->dataType() == INT32) dims.push_back(ax->hostAs<int>()[i * (ax->rankOf() ? ax->strideAt(ax->rankOf() - 1) : 1)]);
      else ND4J_THROW("ArgMax: axis array must be INT32 or INT64");
    }
  }
  return dims;
}
static void argExec(Context& c, int opNum, const char* name) {
  NDArray* x = c.input(0);
  NDArray* z = c.output(0);
  if (z->isEmpty() || z->lengthOf() < 1) return;
  auto raw = argDims(c);
  for (auto d : raw) if (d != 2147483647LL) ND4J_REQUIRE((d < 0 ? d + x->rankOf() : d) < x->rankOf() && (d < 0 ? d + x->rankOf() : d) >= 0, std::string(name) + ": axis can't be above rank");
  auto dims = normalizeDims(x->rankOf(), raw.data(), (LongType)raw.size(), name);
  runIndexReduce(name, opNum, x, z, dims);
}
static std::vector<std::vector<LongType>> argShapeFn(Context& c) {
  NDArray* x = c.input(0);
  DataType dt = c.dArgs.empty() ? INT64 : c.dArgs[0];
  if (x->rankOf() == 0) return {scalarShapeInfo(INT64)};
  auto raw = argDims(c);
  const bool keepDims = bArg(c, 0, false);
  auto dims = normalizeDims(x->rankOf(), raw.data(), (LongType)raw.size(), "ArgMax");
  if (dims.empty()) return {scalarShapeInfo(dt)};
  std::vector<LongType> out;
  for (int d = 0; d < x->rankOf(); d++) {
    bool red = std::find(dims.begin(), dims.end(), (LongType)d) != dims.end();
    if (red) { ND4J_REQUIRE(x->sizeAt(d) != 0, "ArgMax: you can't reduce along axis with 0 in shape"); if (keepDims) out.push_back(1); }
    else out.push_back(x->sizeAt(d));
  }
  return {makeShapeInfo(dt, 'c', out)};
}

static std::vector<LongType> hostIndexVector(NDArray* a, const char* what);
// ---- reduce_* custom ops ----------------------------------------------------------------------------------------------------
// generic/reduce/reduce_sum.cpp:33-61 and its siblings (reduce_max, reduce_min, reduce_prod, reduceMean.cpp, reduce_norm1,
// reduce_norm2, reduce_norm_max, reduce_sqnorm, reduceVariance.cpp, reduceStDev.cpp): dims from IArgs or from a second
// input, keepDims from BArg 0 (or TArg 0), no dims = reduce everything; variance / stdev take biasCorrected from BArg 1
// (or TArg 1).  Thin wrappers over the kernels of the legacy reduce loops, as the reference's are over reduceAlongDimension.
struct ReduceArgs { std::vector<LongType> dims; bool keepDims = false, biasCorrected = false; };
static ReduceArgs reduceArgs(Context& c, const char* name) {
  ReduceArgs r;
  NDArray* x = c.input(0);
  std::vector<LongType> raw = c.width() > 1 ? hostIndexVector(c.input(1), name) : c.iArgs;
  ND4J_REQUIRE((int)raw.size() <= x->rankOf() || x->rankOf() == 0, std::string(name) + ": the number of dimensions to reduce along must be <= input array rank, but got " + std::to_string(raw.size()) + " instead");
  for (auto d : raw)
    ND4J_REQUIRE(d >= -x->rankOf() && d < x->rankOf(), std::string(name) + ": the input dimension to reduce along must be in range [-" + std::to_string(x->rankOf()) + ", " + std::to_string(x->rankOf()) + "), but got " + std::to_string(d) + " instead !");
  r.dims = normalizeDims(x->rankOf(), raw.data(), (LongType)raw.size(), name);
  if (!c.bArgs.empty()) { r.keepDims = c.bArgs[0]; if (c.bArgs.size() > 1) r.biasCorrected = c.bArgs[1]; }
  else if (!c.tArgs.empty()) { r.keepDims = c.tArgs[0] != 0.0; if (c.tArgs.size() > 1) r.biasCorrected = c.tArgs[1] != 0.0; }
  return r;
}
static void reduceCustomExec(Context& c, ReduceKind k, const char* name) {
  ReduceArgs r = reduceArgs(c, name);
  runReduce(name, k, c.input(0), c.output(0), r.dims);
}
static void reduceStatsExec(Context& c, MiscReduceKind k, const char* name) {
  ReduceArgs r = reduceArgs(c, name);
  ND4J_REQUIRE(c.output(0)->dataType() == c.input(0)->dataType() && isFloatType(c.input(0)->dataType()), std::string(name) + ": nd4j-hip requires a floating point input and an output of the same type");
  runReduceMisc(name, k, c.input(0), c.output(0), r.dims, r.biasCorrected);
}
static std::vector<std::vector<LongType>> reduceCustomShapeFn(Context& c, const char* name) {
  NDArray* x = c.input(0);
  ReduceArgs r = reduceArgs(c, name);
  std::vector<LongType> out;
  for (int d = 0; d < x->rankOf(); d++) {
    const bool red = r.dims.empty() || std::find(r.dims.begin(), r.dims.end(), (LongType)d) != r.dims.end();
    if (!red) out.push_back(x->sizeAt(d));
    else if (r.keepDims) out.push_back(1);
  }
  if (out.empty()) return {scalarShapeInfo(x->dataType())};
  return {makeShapeInfo(x->dataType(), x->ordering(), out)};
}

// ---- activation custom ops -------------------------------------------------------------------------------------------------------
// generic/nn/activations/{tanh,sigmoid,softplus,softsign,cube,hardsigmoid,hardtanh,rationaltanh,rectifiedtanh,selu,
// identity}.cpp apply one legacy transform, {relu,relu6,lrelu,elu}.cpp one legacy scalar op whose scalar is TArg 0
// (defaults: relu 0, lrelu 0.01, elu 1); the kernels are those of execTransformStrict / execTransformSame / execScalar.
static void activationExec(Context& c, UnaryKind k, const char* name) {
  NDArray* x = c.input(0); NDArray* z = c.output(0);
  ND4J_REQUIRE(x->dataType() == z->dataType() && isFloatType(x->dataType()), std::string(name) + ": input and output must share a floating point type");
  ND4J_REQUIRE(x->lengthOf() == z->lengthOf(), std::string(name) + ": input and output lengths differ");
  if (x->isEmpty() || z->isEmpty()) return;
  EwPlan p = buildEwPlan({z->shapeInfo(), x->shapeInfo()});
  prepareSpecialUse({z}, {x});
  launchUnary(stream(), k, x->dataType(), z->dataType(), x->specialBuffer(), z->specialBuffer(), p);
  registerSpecialUse({z}, {x});
}
static void scalarActivationExec(Context& c, PairwiseKind k, double defaultScalar, const char* name) {
  NDArray* x = c.input(0); NDArray* z = c.output(0);
  ND4J_REQUIRE(x->dataType() == z->dataType() && isFloatType(x->dataType()), std::string(name) + ": input and output must share a floating point type");
  if (x->isEmpty() || z->isEmpty()) return;
  EwPlan p = buildEwPlan({z->shapeInfo(), x->shapeInfo()});
  ND4J_REQUIRE(p.sameShape, std::string(name) + ": input and output must share a shape");
  prepareSpecialUse({z}, {x});
  launchScalarOp(stream(), k, x->dataType(), x->specialBuffer(), tArg(c, 0, defaultScalar), z->specialBuffer(), p);
  registerSpecialUse({z}, {x});
}

// clipbyvalue (generic/transforms/clip_by_value.cpp:33-83): bounds from TArgs, else from two scalar input arrays
static void clipByValueExec(Context& c) {
  NDArray* x = c.input(0); NDArray* z = c.output(0);
  ND4J_REQUIRE(x->dataType() == z->dataType() && isFloatType(x->dataType()), "clip_by_value: input and output must share a floating point type");
  double left, right;
  if (!c.tArgs.empty()) {
    ND4J_REQUIRE(c.tArgs.size() >= 2, "clip_by_value: two bounds are required");
    left = c.tArgs[0]; right = c.tArgs[1];
    char msg[160];
    std::snprintf(msg, sizeof msg, "clip_by_value: left bound should be lesser than right. But %f >= %f given.", left, right);
    ND4J_REQUIRE(left < right, msg);
  } else {
    ND4J_REQUIRE(c.width() >= 3, "clip_by_value: bounds come as two T arguments or as two scalar inputs");
    NDArray* bounds[2] = {c.input(1), c.input(2)};
    double v[2];
    for (int i = 0; i < 2; i++) {
      ND4J_REQUIRE(isFloatType(bounds[i]->dataType()) && bounds[i]->lengthOf() >= 1, "clip_by_value: a bound must be a floating point scalar");
      bounds[i]->buf->syncToPrimary();
      // the reference reads element 0 as the input's type
      const double raw = hostValueAsDouble(bounds[i]->hostAs<unsigned char>(), bounds[i]->dataType());
      v[i] = x->dataType() == DOUBLE ? raw : (double)(float)raw;
    }
    left = v[0]; right = v[1];
  }
  if (x->isEmpty() || z->isEmpty()) return;
  EwPlan p = buildEwPlan({z->shapeInfo(), x->shapeInfo()});
  ND4J_REQUIRE(p.sameShape, "clip_by_value: input and output must share a shape");
  prepareSpecialUse({z}, {x});
  launchScalar2Op(stream(), S2_CLIP_BY_VALUE, x->dataType(), z->dataType(), x->specialBuffer(), left, right, z->specialBuffer(), p);
  registerSpecialUse({z}, {x});
}

// ---- glue ops for the decode step ----------------------------------------------------------------------------------------------
// gather (generic/transforms/gather.cpp:34): rows of a dense 2-D table picked by an index array, axis 0
static void gatherExec(Context& c) {
  NDArray* table = c.input(0);
  ND4J_REQUIRE(c.width() > 1, "GATHER OP: nd4j-hip takes the indices as the second input array");
  NDArray* idx = c.input(1);
  NDArray* z = c.output(0);
  const LongType axis = iArg(c, 0, 0);
  ND4J_REQUIRE(axis == 0 && table->rankOf() == 2 && table->strideAt(1) == 1 && table->strideAt(0) == table->sizeAt(1),
               "GATHER OP: nd4j-hip implements axis 0 of a dense rank-2 input");
  ND4J_REQUIRE(z->dataType() == table->dataType(), "GATHER OP: output must carry the input's data type");
  ND4J_REQUIRE(z->lengthOf() == idx->lengthOf() * table->sizeAt(1), "GATHER OP: wrong output length");
  EwPlan pz = buildEwPlan({z->shapeInfo(), z->shapeInfo()});
  EwPlan pi = buildEwPlan({idx->shapeInfo(), idx->shapeInfo()});
  ND4J_REQUIRE(pz.contiguous && pi.contiguous, "GATHER OP: indices and output must be dense");
  if (z->isEmpty() || z->lengthOf() == 0) return;
  prepareSpecialUse({z}, {table, idx});
  launchGatherRows(stream(), table->dataType(), idx->dataType(), table->specialBuffer(), idx->specialBuffer(), z->specialBuffer(), idx->lengthOf(), table->sizeAt(1), table->sizeAt(0));
  registerSpecialUse({z}, {table, idx});
}
static std::vector<std::vector<LongType>> gatherShapeFn(Context& c) {
  NDArray* table = c.input(0); NDArray* idx = c.input(1);
  std::vector<LongType> out = shapeOf(idx);
  for (int d = 1; d < table->rankOf(); d++) out.push_back(table->sizeAt(d));
  return {makeShapeInfo(table->dataType(), 'c', out)};
}

// broadcastable add / multiply / subtract / divide (generic/broadcastable/*.cpp, generic/helpers/BroadcastHelper.h:43-66):
// numpy-style broadcasting of y against x realised with zero strides
static std::vector<LongType> broadcastShape(const NDArray* x, const NDArray* y) {
  int r = std::max(x->rankOf(), y->rankOf());
  std::vector<LongType> out(r);
  for (int i = 0; i < r; i++) {
    int xd = i - (r - x->rankOf()), yd = i - (r - y->rankOf());
    LongType xs = xd >= 0 ? x->sizeAt(xd) : 1, ys = yd >= 0 ? y->sizeAt(yd) : 1;
    ND4J_REQUIRE(xs == ys || xs == 1 || ys == 1, "broadcastable op: shapes " + shapeStr(x) + " and " + shapeStr(y) + " do not broadcast");
    out[i] = xs == 1 ? ys : xs;
  }
  return out;
}
static std::vector<LongType> broadcastStrides(const NDArray* a, const std::vector<LongType>& out) {
  int r = (int)out.size();
  std::vector<LongType> st(r, 0);
  for (int i = 0; i < r; i++) {
    int ad = i - (r - a->rankOf());
    if (ad >= 0 && a->sizeAt(ad) != 1) st[i] = a->strideAt(ad);
  }
  return st;
}
static void broadcastableExec(Context& c, PairwiseKind k, const char* name) {
  ND4J_REQUIRE(c.width() >= 2, std::string(name) + ": two inputs are required");
  NDArray* x = c.input(0); NDArray* y = c.input(1); NDArray* z = c.output(0);
  ND4J_REQUIRE(x->dataType() == z->dataType() && y->dataType() == z->dataType() && (isFloatType(z->dataType()) || isIntLike(z->dataType())), std::string(name) + ": nd4j-hip requires inputs and output of one type");
  if (x->isEmpty() || y->isEmpty() || z->isEmpty()) return;
  auto out = broadcastShape(x, y);
  ND4J_REQUIRE(out == shapeOf(z), std::string(name) + ": output shape " + shapeStr(z) + " does not match the broadcast shape");
  auto xs = broadcastStrides(x, out), ys = broadcastStrides(y, out);
  auto xsi = makeShapeInfo(x->dataType(), 'c', out, xs.data()), ysi = makeShapeInfo(y->dataType(), 'c', out, ys.data());
  EwPlan p = buildEwPlan({z->shapeInfo(), xsi.data(), ysi.data()});
  prepareSpecialUse({z}, {x, y});
  launchPairwise(stream(), k, x->dataType(), y->dataType(), z->dataType(), x->specialBuffer(), y->specialBuffer(), z->specialBuffer(), p);
  registerSpecialUse({z}, {x, y});
}
static std::vector<std::vector<LongType>> broadcastableShapeFn(Context& c) {
  NDArray* x = c.input(0); NDArray* y = c.input(1);
  return {makeShapeInfo(x->dataType(), x->ordering(), broadcastShape(x, y))};
}

// biasadd (generic/nn/bias_add.cpp:33-73, alias bias_add; helpers/cpu/addBias.cpp): a rank-1 bias added along the channel
// axis -- the last one, or axis 1 when BArg0 (NCHW) is set; the output carries the bias's data type
static void biasAddExec(Context& c) {
  NDArray* x = c.input(0); NDArray* b = c.input(1); NDArray* z = c.output(0);
  const bool nchw = bArg(c, 0, false);
  const int ch = nchw ? 1 : x->rankOf() - 1;
  ND4J_REQUIRE(b->rankOf() == 1, "BIASADD CUSTOM_OP: bias array should have rank = 1, but got " + std::to_string(b->rankOf()) + " instead !");
  ND4J_REQUIRE(x->rankOf() >= 1 && ch < x->rankOf() && b->sizeAt(0) == x->sizeAt(ch),
               "BIASADD CUSTOM_OP: shapes of bias " + shapeStr(b) + " and input " + shapeStr(x) + " arrays are not suitable for broadcast operation along channel dimension " + std::to_string(ch) + " !");
  ND4J_REQUIRE(shapeOf(z) == shapeOf(x), "BIASADD CUSTOM_OP: wrong shape of output array, expected is " + shapeStr(x) + " but got " + shapeStr(z) + " instead !");
  ND4J_REQUIRE(isFloatType(x->dataType()) && isFloatType(b->dataType()) && isFloatType(z->dataType()), "BIASADD CUSTOM_OP: nd4j-hip implements floating point arrays only");
  if (x->isEmpty() || z->isEmpty()) return;
  std::vector<LongType> bs(x->rankOf(), 0);
  bs[ch] = b->strideAt(0);
  auto bsi = makeShapeInfo(b->dataType(), 'c', shapeOf(x), bs.data());
  EwPlan p = buildEwPlan({z->shapeInfo(), x->shapeInfo(), bsi.data()});
  prepareSpecialUse({z}, {x, b});
  launchPairwise(stream(), P_ADD, x->dataType(), b->dataType(), z->dataType(), x->specialBuffer(), b->specialBuffer(), z->specialBuffer(), p);
  registerSpecialUse({z}, {x, b});
}
static std::vector<std::vector<LongType>> biasAddShapeFn(Context& c) {
  NDArray* x = c.input(0); NDArray* b = c.input(1);
  return {makeShapeInfo(b->dataType(), x->ordering(), shapeOf(x))};
}

// equals, not_equals, greater, greater_equal, less, less_equal (generic/broadcastable/equals.cpp:29-58 and siblings):
// the comparison of the bool tables under broadcasting, BOOL output
static void comparisonExec(Context& c, PairwiseKind k, const char* name) {
  ND4J_REQUIRE(c.width() >= 2, std::string(name) + ": two inputs are required");
  NDArray* x = c.input(0); NDArray* y = c.input(1); NDArray* z = c.output(0);
  ND4J_REQUIRE(z->dataType() == BOOL, std::string(name) + ": the output must be a BOOL array");
  ND4J_REQUIRE(x->dataType() == y->dataType(), std::string(name) + ": nd4j-hip compares arrays of one data type");
  if (x->isEmpty() || y->isEmpty() || z->isEmpty()) return;
  auto out = broadcastShape(x, y);
  ND4J_REQUIRE(out == shapeOf(z), std::string(name) + ": output shape " + shapeStr(z) + " does not match the broadcast shape");
  auto xs = broadcastStrides(x, out), ys = broadcastStrides(y, out);
  auto xsi = makeShapeInfo(x->dataType(), 'c', out, xs.data()), ysi = makeShapeInfo(y->dataType(), 'c', out, ys.data());
  EwPlan p = buildEwPlan({z->shapeInfo(), xsi.data(), ysi.data()});
  prepareSpecialUse({z}, {x, y});
  launchPairwise(stream(), k, x->dataType(), y->dataType(), BOOL, x->specialBuffer(), y->specialBuffer(), z->specialBuffer(), p);
  registerSpecialUse({z}, {x, y});
}
static std::vector<std::vector<LongType>> comparisonShapeFn(Context& c) {
  NDArray* x = c.input(0); NDArray* y = c.input(1);
  return {makeShapeInfo(BOOL, x->ordering(), broadcastShape(x, y))};
}

// zeros_as (aliases zeroslike, zeros_like) and ones_as (generic/tensor/zeros_as.cpp:30-60, ones_as.cpp): an array of the
// input's shape, of the type named by DArg0 (default: the input's), filled with 0 / 1
static void fillAsExec(Context& c, double v, const char* name) {
  NDArray* z = c.output(0);
  if (z->isEmpty()) return;
  ND4J_REQUIRE(isFloatType(z->dataType()), std::string(name) + ": nd4j-hip fills floating point arrays only");
  prepareSpecialUse({z}, {});
  fillValue(z, v);
  registerSpecialUse({z}, {});
}
static std::vector<std::vector<LongType>> fillAsShapeFn(Context& c) {
  NDArray* x = c.input(0);
  const DataType dt = c.dArgs.empty() ? x->dataType() : c.dArgs[0];
  return {makeShapeInfo(dt, x->ordering(), shapeOf(x))};
}

// concat (generic/transforms/concat.cpp:34): inputs joined along IArg0 (or the last input when BArg0 is set)
static void concatExec(Context& c) {
  int n = c.width();
  ND4J_REQUIRE(n >= 1, "CONCAT OP: at least one input is required");
  LongType axis;
  if (bArg(c, 0, false)) {
    NDArray* ax = c.input(n - 1);
    ax->buf->syncToPrimary();
    axis = ax->dataType() == INT64 ? ax->hostAs<LongType>()[0] : ax->hostAs<int>()[0];
    n--;
  } else axis = iArg(c, 0, 0);
  NDArray* z = c.output(0);
  const int rank = z->rankOf();
  if (axis < 0) axis += rank;
  ND4J_REQUIRE(axis >= 0 && axis < rank, "CONCAT OP: axis out of range");
  std::vector<NDArray*> reads;
  LongType total = 0;
  for (int i = 0; i < n; i++) {
    NDArray* a = c.input(i);
    if (a->isEmpty()) continue;
    ND4J_REQUIRE(a->rankOf() == rank && a->dataType() == z->dataType(), "CONCAT OP: inputs must share rank and data type with the output");
    for (int d = 0; d < rank; d++) if (d != axis) ND4J_REQUIRE(a->sizeAt(d) == z->sizeAt(d), "CONCAT OP: input shapes differ outside the concat axis");
    total += a->sizeAt((int)axis);
    reads.push_back(a);
  }
  ND4J_REQUIRE(total == z->sizeAt((int)axis), "CONCAT OP: output extent along the axis does not match the inputs");
  prepareSpecialUse(std::vector<NDArray*>{z}, reads);
  LongType at = 0;
  for (NDArray* a : reads) {
    // view of z covering this input's slot
    std::vector<LongType> shp = shapeOf(a), st(rank);
    for (int d = 0; d < rank; d++) st[d] = z->strideAt(d);
    auto vsi = makeShapeInfo(z->dataType(), 'c', shp, st.data());
    EwPlan p = buildEwPlan({vsi.data(), a->shapeInfo()});
    char* dst = (char*)z->specialBuffer() + (size_t)(at * z->strideAt((int)axis)) * sizeOf(z->dataType());
    launchUnary(stream(), U_IDENTITY, a->dataType(), z->dataType(), a->specialBuffer(), dst, p);
    at += a->sizeAt((int)axis);
  }
  registerSpecialUse(std::vector<NDArray*>{z}, reads);
}
static std::vector<std::vector<LongType>> concatShapeFn(Context& c) {
  int n = c.width();
  LongType axis = iArg(c, 0, 0);
  if (bArg(c, 0, false)) { NDArray* ax = c.input(n - 1); ax->buf->syncToPrimary(); axis = ax->dataType() == INT64 ? ax->hostAs<LongType>()[0] : ax->hostAs<int>()[0]; n--; }
  NDArray* first = c.input(0);
  std::vector<LongType> out = shapeOf(first);
  if (axis < 0) axis += first->rankOf();
  ND4J_REQUIRE(axis >= 0 && axis < first->rankOf(), "CONCAT OP: axis out of range");
  out[axis] = 0;
  for (int i = 0; i < n; i++) if (!c.input(i)->isEmpty()) out[axis] += c.input(i)->sizeAt((int)axis);
  return {makeShapeInfo(first->dataType(), 'c', out)};
}

// ---- shape ops: every one of them is "z = a view of x, enumerated in some order" -------------------------------------------------
// integer arguments that may come as IArgs or as an integer input array
static std::vector<LongType> hostIndexVector(NDArray* a, const char* what) {
  std::vector<LongType> out;
  if (!a || a->isEmpty() || a->lengthOf() == 0) return out;
  ND4J_REQUIRE(a->buf, std::string(what) + ": index array has no buffer");
  a->buf->syncToPrimary();
  out.resize(a->lengthOf());
  for (LongType i = 0; i < (LongType)out.size(); i++) {
    LongType off = 0, idx = i;
    for (int d = a->rankOf() - 1; d >= 0; d--) { off += (idx % a->sizeAt(d)) * a->strideAt(d); idx /= a->sizeAt(d); }
    if (a->dataType() == INT64) out[i] = a->hostAs<LongType>()[off];
    else if (a->dataType() == INT32) out[i] = a->hostAs<int>()[off];
    else ND4J_THROW(std::string(what) + ": index array must be INT32 or INT64");
  }
  return out;
}
static bool denseIn(const std::vector<LongType>& shape, const std::vector<LongType>& stride) {   // row-major without gaps
  LongType expect = 1;
  for (int d = (int)shape.size() - 1; d >= 0; d--) {
    if (shape[d] != 1 && stride[d] != expect) return false;
    expect *= shape[d];
  }
  return true;
}
// z[i-th element] = view[i-th element], both enumerated row-major over their own shapes (column-major for order 'f');
// the view is (src + srcOffsetElems, shape, strides) over x's buffer
static void assignEnumerated(NDArray* z, NDArray* x, LongType srcOffsetElems, std::vector<LongType> vshape, std::vector<LongType> vstride,
                             char order, const char* name) {
  ND4J_REQUIRE(z->dataType() == x->dataType(), std::string(name) + ": output must carry the input's data type");
  LongType n = 1;
  for (auto v : vshape) n *= v;
  ND4J_REQUIRE(n == z->lengthOf(), std::string(name) + ": output length " + std::to_string(z->lengthOf()) + " does not match " + std::to_string(n));
  if (n == 0) return;
  std::vector<LongType> zshape = shapeOf(z), zstride(z->rankOf());
  for (int d = 0; d < z->rankOf(); d++) zstride[d] = z->strideAt(d);
  if (order == 'f') {
    std::reverse(vshape.begin(), vshape.end()); std::reverse(vstride.begin(), vstride.end());
    std::reverse(zshape.begin(), zshape.end()); std::reverse(zstride.begin(), zstride.end());
  }
  if (vshape.empty()) { vshape = {1}; vstride = {1}; }
  if (zshape.empty()) { zshape = {1}; zstride = {1}; }
  if (denseIn(vshape, vstride) && denseIn(zshape, zstride)) {   // both flat: one contiguous copy
    vshape = zshape = {n};
    vstride = zstride = {1};
  }
  auto vsi = makeShapeInfo(x->dataType(), 'c', vshape, vstride.data());
  auto zsi = makeShapeInfo(z->dataType(), 'c', zshape, zstride.data());
  EwPlan p = buildEwPlan({zsi.data(), vsi.data()});
  prepareSpecialUse({z}, {x});
  const char* src = (const char*)x->specialBuffer() + (size_t)srcOffsetElems * sizeOf(x->dataType());
  launchUnary(stream(), U_IDENTITY, x->dataType(), z->dataType(), src, z->specialBuffer(), p);
  registerSpecialUse({z}, {x});
}
static std::vector<LongType> stridesOf(const NDArray* a) {
  std::vector<LongType> st(a->rankOf());
  for (int d = 0; d < a->rankOf(); d++) st[d] = a->strideAt(d);
  return st;
}

// permute (generic/shape/permute.cpp:35-63) and transpose (generic/shape/transpose.cpp:33-77): z = dense copy of the permuted view;
// the permutation comes from the IArgs or a second input, none = reversed axes
static std::vector<LongType> permutationOf(Context& c, const char* name) {
  NDArray* x = c.input(0);
  std::vector<LongType> perm = c.width() > 1 ? hostIndexVector(c.input(1), name) : c.iArgs;
  const int r = x->rankOf();
  if (perm.empty()) { perm.resize(r); for (int i = 0; i < r; i++) perm[i] = r - 1 - i; return perm; }
  ND4J_REQUIRE((int)perm.size() == r, std::string(name) + ": number of permutations is less in size than input rank.");
  std::vector<bool> seen(r, false);
  for (auto& v : perm) {
    if (v < 0) v += r;
    ND4J_REQUIRE(v >= 0 && v < r && !seen[v], std::string(name) + ": not a permutation of the input's axes");
    seen[v] = true;
  }
  return perm;
}
static void permuteExec(Context& c, const char* name) {
  NDArray* x = c.input(0); NDArray* z = c.output(0);
  if (x->isEmpty()) { ND4J_REQUIRE(z->isEmpty(), std::string(name) + ": when input is empty, output must also be empty"); return; }
  auto perm = permutationOf(c, name);
  std::vector<LongType> shp(perm.size()), st(perm.size());
  for (size_t i = 0; i < perm.size(); i++) { shp[i] = x->sizeAt((int)perm[i]); st[i] = x->strideAt((int)perm[i]); }
  ND4J_REQUIRE(shp == shapeOf(z), std::string(name) + ": output shape " + shapeStr(z) + " is not the permuted input shape");
  assignEnumerated(z, x, 0, shp, st, 'c', name);
}
static std::vector<std::vector<LongType>> permuteShapeFn(Context& c, const char* name) {
  NDArray* x = c.input(0);
  if (x->rankOf() < 1) return {scalarShapeInfo(x->dataType())};
  auto perm = permutationOf(c, name);
  std::vector<LongType> shp(perm.size());
  for (size_t i = 0; i < perm.size(); i++) shp[i] = x->sizeAt((int)perm[i]);
  return {makeShapeInfo(x->dataType(), 'c', shp)};
}

// reshape (generic/shape/reshape.cpp:33-71,174-260): shape from the IArgs ({-order, dims...}, order -99 = 'c', -102 = 'f') or from a
// second input; one -1 is inferred; the data keeps its sequence in the chosen order
static std::vector<LongType> reshapeTarget(Context& c, char& order) {
  NDArray* x = c.input(0);
  std::vector<LongType> args = c.width() > 1 ? hostIndexVector(c.input(1), "Reshape") : c.iArgs;
  order = 'c';
  if (!args.empty() && args[0] < 0 && args[0] != -1) {
    ND4J_REQUIRE(args[0] == -99 || args[0] == -102, "reshape:: Value passed in must be -99 or -102 for the ordering if an int array is present.");
    order = (char)(-args[0]);
    args.erase(args.begin());
  }
  if (c.width() > 1 && !c.iArgs.empty() && (c.iArgs[0] == 99 || c.iArgs[0] == 102 || c.iArgs[0] == -99 || c.iArgs[0] == -102))
    order = (char)std::abs(c.iArgs[0]);
  LongType known = 1; int pos = -1;
  for (size_t i = 0; i < args.size(); i++) {
    if (args[i] == -1) { ND4J_REQUIRE(pos == -1, "Reshape : Only one unknown dimension (-1) is allowed."); pos = (int)i; }
    else { ND4J_REQUIRE(args[i] >= 0, "Reshape: negative dimension"); known *= args[i]; }
  }
  if (pos >= 0) {
    if (x->lengthOf() == 1 && x->rankOf() <= 1) args[pos] = 1;
    else { ND4J_REQUIRE(known > 0 && x->lengthOf() % known == 0, "Reshape: the unknown dimension cannot be resolved"); args[pos] = x->lengthOf() / known; }
  }
  return args;
}
static void reshapeExec(Context& c) {
  NDArray* x = c.input(0); NDArray* z = c.output(0);
  if (x->isEmpty()) { ND4J_REQUIRE(z->isEmpty(), "Reshape: when input is empty, output must also be empty"); return; }
  ND4J_REQUIRE(x->lengthOf() == z->lengthOf(), "Reshape: lengths before and after reshape should match, but got " + std::to_string(x->lengthOf()) + " vs " + std::to_string(z->lengthOf()));
  ND4J_REQUIRE(z->ordering() == 'c' || z->ordering() == 'f', "Reshape: new shape has unknown order");
  assignEnumerated(z, x, 0, shapeOf(x), stridesOf(x), z->ordering(), "Reshape");
}
static std::vector<std::vector<LongType>> reshapeShapeFn(Context& c) {
  char order;
  auto shp = reshapeTarget(c, order);
  NDArray* x = c.input(0);
  if (shp.empty()) return {scalarShapeInfo(x->dataType())};
  return {makeShapeInfo(x->dataType(), order, shp)};
}

// squeeze (generic/shape/squeeze.cpp:32-78) / expand_dims (generic/shape/expand_dims.cpp:32-50): same data in the input's order
static std::vector<LongType> squeezedShape(Context& c) {
  NDArray* x = c.input(0);
  std::vector<LongType> axis = !c.iArgs.empty() ? c.iArgs : (c.width() > 1 ? hostIndexVector(c.input(1), "squeeze") : std::vector<LongType>{});
  for (auto& a : axis) if (a < 0) a += x->rankOf();
  std::vector<LongType> shp;
  for (int d = 0; d < x->rankOf(); d++) {
    if (x->sizeAt(d) == 1 && (axis.empty() || std::find(axis.begin(), axis.end(), (LongType)d) != axis.end())) continue;
    shp.push_back(x->sizeAt(d));
  }
  return shp;
}
static void sameDataExec(Context& c, const char* name) {
  NDArray* x = c.input(0); NDArray* z = c.output(0);
  if (x->isEmpty()) return;
  assignEnumerated(z, x, 0, shapeOf(x), stridesOf(x), x->ordering() == 'f' && z->ordering() == 'f' ? 'f' : 'c', name);
}
static std::vector<std::vector<LongType>> squeezeShapeFn(Context& c) {
  NDArray* x = c.input(0);
  if (x->rankOf() == 0 || (x->rankOf() == 1 && x->lengthOf() == 1)) return {scalarShapeInfo(x->dataType())};
  return {makeShapeInfo(x->dataType(), x->ordering(), squeezedShape(c))};
}
static std::vector<std::vector<LongType>> expandDimsShapeFn(Context& c) {
  NDArray* x = c.input(0);
  if (x->lengthOf() == 1 && x->rankOf() <= 1 && !x->isEmpty())
    return {makeShapeInfo(x->dataType(), 'c', x->rankOf() < 1 ? std::vector<LongType>{1} : std::vector<LongType>{1, 1})};
  LongType axis = !c.iArgs.empty() ? c.iArgs[0] : hostIndexVector(c.input(1), "ExpandDims").at(0);
  if (axis < 0) axis += x->rankOf() + 1;
  ND4J_REQUIRE(axis >= 0 && axis <= x->rankOf(), "ExpandDims: axis should be in range of 0..." + std::to_string(x->rankOf() + 1) + " in this case, but got " + std::to_string(axis) + " instead");
  std::vector<LongType> shp = shapeOf(x);
  shp.insert(shp.begin() + axis, 1);
  return {makeShapeInfo(x->dataType(), x->ordering(), shp)};
}

// split (generic/transforms/split.cpp:32-72): IArg0 equal parts along the axis (IArg1, or a scalar input before/after the array)
static NDArray* splitInput(Context& c, LongType& axis) {
  NDArray* x = c.input(0);
  axis = 0;
  if (c.width() > 1) {
    NDArray* a = c.input(0); NDArray* b = c.input(1);
    if (a->lengthOf() == 1 && a->rankOf() == 0) { axis = hostIndexVector(a, "Split").at(0); x = b; }
    else if (b->lengthOf() == 1 && b->rankOf() == 0) { axis = hostIndexVector(b, "Split").at(0); x = a; }
  }
  if (c.iArgs.size() == 2) axis = c.iArgs[1];
  if (axis < 0) axis += x->rankOf();
  return x;
}
static void splitExec(Context& c) {
  ND4J_REQUIRE(!c.iArgs.empty(), "Split: num_splits is required as the first integer argument");
  const LongType parts = c.iArgs[0];
  LongType axis;
  NDArray* x = splitInput(c, axis);
  if (x->isEmpty()) return;
  ND4J_REQUIRE(axis >= 0 && axis < x->rankOf(), "Split: axis out of range");
  ND4J_REQUIRE(parts > 0 && x->sizeAt((int)axis) % parts == 0, "Split: num_splits has wrong value, remainder of division should be 0, but it's " +
                                                                    std::to_string(parts > 0 ? x->sizeAt((int)axis) % parts : -1));
  ND4J_REQUIRE((LongType)c.outputs.size() >= parts, "Split: " + std::to_string(parts) + " output arrays are required");
  std::vector<LongType> shp = shapeOf(x);
  shp[axis] /= parts;
  for (LongType i = 0; i < parts; i++) {
    NDArray* z = c.output((int)i);
    ND4J_REQUIRE(z && shapeOf(z) == shp, "Split: output " + std::to_string(i) + " has the wrong shape");
    assignEnumerated(z, x, i * shp[axis] * x->strideAt((int)axis), shp, stridesOf(x), 'c', "Split");
  }
}
static std::vector<std::vector<LongType>> splitShapeFn(Context& c) {
  ND4J_REQUIRE(!c.iArgs.empty(), "Split: num_splits is required as the first integer argument");
  const LongType parts = c.iArgs[0];
  LongType axis;
  NDArray* x = splitInput(c, axis);
  ND4J_REQUIRE(axis >= 0 && axis < x->rankOf() && parts > 0, "Split: axis or num_splits out of range");
  std::vector<LongType> shp = shapeOf(x);
  shp[axis] /= parts;
  std::vector<std::vector<LongType>> out;
  for (LongType i = 0; i < parts; i++) out.push_back(makeShapeInfo(x->dataType(), x->ordering(), shp));
  return out;
}

// unstack (generic/transforms/unstack.cpp:32-108): one output per index along IArg0, each the input with that axis removed
// (a vector falls apart into scalars)
static std::vector<LongType> unstackShape(NDArray* x, LongType dim) {
  std::vector<LongType> shp;
  for (int d = 0; d < x->rankOf(); d++) if (d != dim) shp.push_back(x->sizeAt(d));
  return shp;
}
static LongType unstackDim(Context& c, NDArray* x) {
  ND4J_REQUIRE(!c.iArgs.empty(), "Unstack: the dimension is required as the first integer argument");
  LongType dim = c.iArgs[0];
  if (dim < 0) dim += x->rankOf();
  ND4J_REQUIRE(dim < x->rankOf(), "Unstack dimension should be lower then rank of input " + std::to_string(x->rankOf()) + ", but got dimension=" + std::to_string(dim) + " !");
  ND4J_REQUIRE(dim >= 0, "Unstack dimension should be non-negative value, but got " + std::to_string(dim) + " !");
  return dim;
}
static void unstackExec(Context& c) {
  NDArray* x = c.input(0);
  if (x->isEmpty()) return;
  const LongType dim = unstackDim(c, x);
  const LongType n = x->sizeAt((int)dim);
  ND4J_REQUIRE((LongType)c.outputs.size() >= n, "Unstack: " + std::to_string(n) + " output arrays are required");
  std::vector<LongType> shp, st;
  for (int d = 0; d < x->rankOf(); d++) if (d != dim) { shp.push_back(x->sizeAt(d)); st.push_back(x->strideAt(d)); }
  for (LongType i = 0; i < n; i++) assignEnumerated(c.output((int)i), x, i * x->strideAt((int)dim), shp, st, 'c', "Unstack");
}
static std::vector<std::vector<LongType>> unstackShapeFn(Context& c) {
  NDArray* x = c.input(0);
  const LongType dim = unstackDim(c, x);
  const LongType n = c.iArgs.size() > 1 ? c.iArgs[1] : x->sizeAt((int)dim);
  std::vector<LongType> shp = unstackShape(x, dim);
  std::vector<std::vector<LongType>> out;
  for (LongType i = 0; i < n; i++) out.push_back(shp.empty() ? scalarShapeInfo(x->dataType()) : makeShapeInfo(x->dataType(), x->ordering(), shp));
  return out;
}

// stack (generic/transforms/stack.cpp:31-92; aliases pack, Pack): equal-shaped inputs side by side along a new axis IArg0
static LongType stackDim(Context& c, NDArray* first) {
  LongType dim = iArg(c, 0, 0);
  if (dim < 0) dim += first->rankOf() + 1;
  ND4J_REQUIRE(dim >= 0 && dim <= first->rankOf(), "STACK op: the input dimension parameter must be <= rank of input arrays shapes (rank=" +
               std::to_string(first->rankOf()) + "), but got " + std::to_string(dim) + " instead !");
  return dim;
}
static void stackExec(Context& c) {
  NDArray* first = c.input(0); NDArray* z = c.output(0);
  const LongType dim = stackDim(c, first);
  if (z->isEmpty()) return;
  const int n = c.width();
  for (int i = 0; i + 1 < n; i++)
    ND4J_REQUIRE(shapeOf(c.input(i)) == shapeOf(c.input(i + 1)), "STACK op: the shapes of all input arrays must be the same !");
  if (first->isEmpty()) return;
  ND4J_REQUIRE(z->rankOf() == first->rankOf() + 1 && z->sizeAt((int)dim) == n && z->dataType() == first->dataType(), "STACK op: wrong output array");
  std::vector<LongType> shp = shapeOf(first), zst;
  for (int d = 0; d < z->rankOf(); d++) if (d != dim) zst.push_back(z->strideAt(d));
  std::vector<NDArray*> reads;
  for (int i = 0; i < n; i++) reads.push_back(c.input(i));
  prepareSpecialUse(std::vector<NDArray*>{z}, reads);
  for (int i = 0; i < n; i++) {
    NDArray* a = c.input(i);
    std::vector<LongType> vshape = shp, vstride = zst;
    if (vshape.empty()) { vshape = {1}; vstride = {1}; }
    auto vsi = makeShapeInfo(z->dataType(), 'c', vshape, vstride.data());
    std::vector<LongType> ashape = shapeOf(a), astride = stridesOf(a);
    if (ashape.empty()) { ashape = {1}; astride = {1}; }
    auto asi = makeShapeInfo(a->dataType(), 'c', ashape, astride.data());
    EwPlan p = buildEwPlan({vsi.data(), asi.data()});
    char* dst = (char*)z->specialBuffer() + (size_t)(i * z->strideAt((int)dim)) * sizeOf(z->dataType());
    launchUnary(stream(), U_IDENTITY, a->dataType(), z->dataType(), a->specialBuffer(), dst, p);
  }
  registerSpecialUse(std::vector<NDArray*>{z}, reads);
}
static std::vector<std::vector<LongType>> stackShapeFn(Context& c) {
  NDArray* first = c.input(0);
  const LongType dim = stackDim(c, first);
  std::vector<LongType> out = shapeOf(first);
  out.insert(out.begin() + dim, (LongType)c.width());
  return {makeShapeInfo(first->dataType(), first->ordering(), out)};
}

// cast (generic/datatypes/cast.cpp:30-86; alias Cast): assignment into an array of the type named by DArg0 or IArg0
static void castExec(Context& c) {
  NDArray* x = c.input(0); NDArray* z = c.output(0);
  if (x->isEmpty()) { ND4J_REQUIRE(z->isEmpty(), "If input is empty, output array must also be empty"); return; }
  if (z == x) return;
  ND4J_REQUIRE(z->lengthOf() == x->lengthOf(), "cast: output must have the input's length");
  EwPlan p = buildEwPlan({z->shapeInfo(), x->shapeInfo()});
  prepareSpecialUse({z}, {x});
  launchUnary(stream(), U_IDENTITY, x->dataType(), z->dataType(), x->specialBuffer(), z->specialBuffer(), p);
  registerSpecialUse({z}, {x});
}
static std::vector<std::vector<LongType>> castShapeFn(Context& c) {
  NDArray* x = c.input(0);
  DataType dt;
  if (!c.dArgs.empty()) dt = c.dArgs[0];
  else { ND4J_REQUIRE(!c.iArgs.empty(), "cast: the new data type is required as a D or I argument"); dt = (DataType)c.iArgs[0]; }
  ND4J_REQUIRE(sizeOf(dt) > 0, "cast: new data type " + std::to_string((int)dt) + " is not supported by nd4j-hip");
  return {makeShapeInfo(dt, x->ordering(), shapeOf(x))};
}

// integer arguments given as an input array of any numeric type (the reference reads them with asVectorT<LongType>)
static std::vector<LongType> hostNumbersAsLong(NDArray* a, const char* what) {
  if (a->dataType() == INT32 || a->dataType() == INT64) return hostIndexVector(a, what);
  std::vector<LongType> out;
  if (a->isEmpty() || a->lengthOf() == 0) return out;
  ND4J_REQUIRE(isFloatType(a->dataType()), std::string(what) + ": a numeric array is required");
  a->buf->syncToPrimary();
  for (LongType i = 0; i < a->lengthOf(); i++) {
    const LongType off = a->rankOf() == 0 ? 0 : i * a->strideAt(a->rankOf() - 1);
    out.push_back((LongType)hostValueAsDouble(a->hostAs<unsigned char>() + off * sizeOf(a->dataType()), a->dataType()));
  }
  return out;
}

// tile (generic/transforms/tile.cpp:31-108): the input repeated reps[d] times along every axis d; reps from IArgs (one per
// axis) or from a second input
static std::vector<LongType> tileReps(Context& c) {
  NDArray* x = c.input(0);
  std::vector<LongType> reps;
  if ((int)c.iArgs.size() == x->rankOf()) reps = c.iArgs;
  else if (c.width() > 1) {
    reps = hostNumbersAsLong(c.input(1), "TILE op");
    ND4J_REQUIRE((int)reps.size() == x->rankOf(), "TILE op: repeats vector length should be equal to input rank, but got " + std::to_string(reps.size()) + " and " + std::to_string(x->rankOf()) + " correspondingly !");
  } else ND4J_THROW("TILE op: this op requires repeats vector, either as IArgs or second array with length equal to rank of input array to be tiled !");
  LongType prod = 1;
  for (auto r : reps) prod *= r;
  ND4J_REQUIRE(prod > 0, "TILE op: reps can't contain 0s");
  return reps;
}
static void tileExec(Context& c) {
  NDArray* x = c.input(0); NDArray* z = c.output(0);
  auto reps = tileReps(c);
  const int rank = x->rankOf();
  ND4J_REQUIRE(z->rankOf() == rank && z->dataType() == x->dataType(), "TILE op: wrong output array");
  // z seen as [reps0, n0, reps1, n1, ...] and x as the same shape with stride 0 along the repeat axes
  std::vector<LongType> shp, zs, xs;
  for (int d = 0; d < rank; d++) {
    ND4J_REQUIRE(z->sizeAt(d) == x->sizeAt(d) * reps[d], "TILE op: wrong output shape");
    shp.push_back(reps[d]); zs.push_back(x->sizeAt(d) * z->strideAt(d)); xs.push_back(0);
    shp.push_back(x->sizeAt(d)); zs.push_back(z->strideAt(d)); xs.push_back(x->strideAt(d));
  }
  if (x->isEmpty() || z->isEmpty() || x->lengthOf() == 0) return;
  if (shp.empty()) { shp = {1}; zs = {1}; xs = {1}; }
  auto zsi = makeShapeInfo(z->dataType(), 'c', shp, zs.data()), xsi = makeShapeInfo(x->dataType(), 'c', shp, xs.data());
  EwPlan p = buildEwPlan({zsi.data(), xsi.data()});
  prepareSpecialUse({z}, {x});
  launchUnary(stream(), U_IDENTITY, x->dataType(), z->dataType(), x->specialBuffer(), z->specialBuffer(), p);
  registerSpecialUse({z}, {x});
}
static std::vector<std::vector<LongType>> tileShapeFn(Context& c) {
  NDArray* x = c.input(0);
  auto reps = tileReps(c);
  std::vector<LongType> out = shapeOf(x);
  for (int d = 0; d < x->rankOf(); d++) out[d] *= reps[d];
  return {makeShapeInfo(x->dataType(), x->ordering(), out)};
}

// slice (generic/transforms/slice.cpp:31-120): begin and size per axis (size -1 = to the end), from IArgs
// [begin.., size..] or from two input arrays
struct SliceArgs { std::vector<LongType> begin, size; bool empty = false; };
static SliceArgs sliceArgs(Context& c) {
  NDArray* x = c.input(0);
  const int rank = x->rankOf();
  SliceArgs a;
  if (c.width() == 3) { a.begin = hostNumbersAsLong(c.input(1), "Slice"); a.size = hostNumbersAsLong(c.input(2), "Slice"); }
  else {
    ND4J_REQUIRE((int)c.iArgs.size() >= 2 * rank, "Number of IArgs should be equal to [" + std::to_string(2 * rank) + "] but got [" + std::to_string(c.iArgs.size()) + "] instead");
    a.begin.assign(c.iArgs.begin(), c.iArgs.begin() + rank);
    a.size.assign(c.iArgs.begin() + rank, c.iArgs.begin() + 2 * rank);
  }
  ND4J_REQUIRE((int)a.begin.size() == rank, "begin array should have length of [" + std::to_string(rank) + "] but got [" + std::to_string(a.begin.size()) + "] instead");
  ND4J_REQUIRE((int)a.size.size() == rank, "size array should have length of [" + std::to_string(rank) + "] but got [" + std::to_string(a.size.size()) + "] instead");
  for (int d = 0; d < rank; d++) {
    const LongType start = a.begin[d];
    ND4J_REQUIRE(start >= 0, "Slice: start index should not be negative");
    ND4J_REQUIRE(start <= x->sizeAt(d), "Index " + std::to_string(start) + " is invalid for dimension " + std::to_string(d) + " with size " + std::to_string(x->sizeAt(d)) + ".");
    if (a.size[d] == -1) a.size[d] = x->sizeAt(d) - start;
    ND4J_REQUIRE(a.size[d] >= 0, "Slice: interval for dimension " + std::to_string(d) + " is less then 1");
    ND4J_REQUIRE(start + a.size[d] <= x->sizeAt(d), "Slice: interval [" + std::to_string(start) + ", " + std::to_string(start + a.size[d]) + "] is out of bounds for dimension " +
                 std::to_string(d) + " with size " + std::to_string(x->sizeAt(d)));
    if (start == x->sizeAt(d) || a.size[d] == 0) a.empty = true;
  }
  return a;
}
static void sliceExec(Context& c) {
  NDArray* x = c.input(0); NDArray* z = c.output(0);
  SliceArgs a = sliceArgs(c);
  if (a.empty || x->isEmpty() || z->isEmpty()) return;
  ND4J_REQUIRE(shapeOf(z) == a.size, "Slice: output shape " + shapeStr(z) + " does not match the requested sizes");
  LongType off = 0;
  for (int d = 0; d < x->rankOf(); d++) off += a.begin[d] * x->strideAt(d);
  assignEnumerated(z, x, off, a.size, stridesOf(x), 'c', "Slice");
}
static std::vector<std::vector<LongType>> sliceShapeFn(Context& c) {
  NDArray* x = c.input(0);
  SliceArgs a = sliceArgs(c);
  return {makeShapeInfo(x->dataType(), 'c', a.size)};
}

// strided_slice (generic/tensor/strided_slice.cpp:135-370,372-530): IArgs = begin_mask, ellipsis_mask, end_mask, new_axis_mask,
// shrink_axis_mask [, begin.., end.., strides..]; or begin/end/strides as inputs 1..3.  The sparse specification (one entry per
// written index) is spread over the input's axes, every axis gets a canonical [begin, end) and a step, and the output is the
// strided view copied out, with new axes inserted and shrunk axes dropped.
struct SliceGeometry {
  std::vector<LongType> begin, count, step;   // per input axis
  std::vector<LongType> outShape;
  bool empty = false;
};
static SliceGeometry sliceGeometry(Context& c) {
  NDArray* x = c.input(0);
  ND4J_REQUIRE(c.iArgs.size() >= 5, "StridedSlice: five mask arguments are required");
  const LongType beginMask = c.iArgs[0], ellipsisMaskIn = c.iArgs[1], endMask = c.iArgs[2], newAxisMask = c.iArgs[3], shrinkMask = c.iArgs[4];
  std::vector<LongType> b, e, st;
  if (c.iArgs.size() > 5) {
    const size_t vals = c.iArgs.size() - 5;
    ND4J_REQUIRE(vals % 3 == 0, "StridedSlice: Number of Integer arguments should be equal to input rank x 3 = " + std::to_string(x->rankOf() * 3) + ", but got " + std::to_string(vals) + " instead");
    const size_t n = vals / 3;
    b.assign(c.iArgs.begin() + 5, c.iArgs.begin() + 5 + n);
    e.assign(c.iArgs.begin() + 5 + n, c.iArgs.begin() + 5 + 2 * n);
    st.assign(c.iArgs.begin() + 5 + 2 * n, c.iArgs.end());
  } else if (c.width() > 1) {
    ND4J_REQUIRE(c.width() >= 3, "StridedSlice: begin and end inputs are required");
    auto asLong = [](NDArray* a) {
      std::vector<LongType> out;
      if (!a || a->lengthOf() == 0) return out;
      if (a->dataType() == INT32 || a->dataType() == INT64) return hostIndexVector(a, "StridedSlice");
      a->buf->syncToPrimary();   // the reference's tests also pass these as float / double arrays
      out.resize(a->lengthOf());
      for (LongType i = 0; i < (LongType)out.size(); i++) {
        const LongType off = a->rankOf() == 0 ? 0 : i * a->strideAt(a->rankOf() - 1);
        if (a->dataType() == FLOAT32) out[i] = (LongType)a->hostAs<float>()[off];
        else if (a->dataType() == DOUBLE) out[i] = (LongType)a->hostAs<double>()[off];
        else ND4J_THROW("StridedSlice: begin/end/strides must be integer, float or double arrays");
      }
      return out;
    };
    b = asLong(c.input(1)); e = asLong(c.input(2));
    ND4J_REQUIRE(b.size() == e.size(), "StridedSlice: Length of begin/end should match, but got " + std::to_string(b.size()) + " vs " + std::to_string(e.size()) + " instead");
    for (size_t i = 0; i < e.size(); i++)   // negative ends count from the end of the axis with the same position (strided_slice.cpp:424-436)
      if (e[i] < 0 && (int)i < x->rankOf()) e[i] = e[i] == -1 ? x->sizeAt((int)i) : e[i] + x->sizeAt((int)i);
    if (c.width() > 3) {
      st = asLong(c.input(3));
      ND4J_REQUIRE(st.size() == b.size(), "StridedSlice: Length of begin/end/stride should match");
    } else st.assign(b.size(), 1);
  } else ND4J_THROW("StridedSlice: Can't find begin/end/stride information neither in IArguments or in input arrays");
  const int n = (int)st.size(), rank = x->rankOf();
  ND4J_REQUIRE(n > 0, "Strided_Slice: empty arguments");
  if (rank == 0) return SliceGeometry{};   // a scalar stays a scalar (strided_slice.cpp:519-522)
  for (auto v : st) ND4J_REQUIRE(v != 0, "StridedSlice: zero stride");

  // spread the sparse specification over the input's axes
  LongType ellipsisMask = ellipsisMaskIn;
  int sparseDims = n, axesAfterEllipsis = 0;
  bool seen = false;
  for (int i = 0; i < n; i++) {
    if (seen && (newAxisMask >> i & 1)) axesAfterEllipsis++;
    if (ellipsisMask >> i & 1) seen = true;
  }
  if (!seen) { ellipsisMask |= 1LL << n; sparseDims++; }
  std::vector<LongType> db(rank, 0), de(rank, 0), ds(rank, 1);
  std::vector<bool> mb(rank, false), me(rank, false), shrink(rank, false);
  std::vector<int> gather;   // per output axis: input axis, -1 shrunk away, -2 new axis
  int full = 0;
  for (int i = 0; i < sparseDims; i++) {
    if (ellipsisMask >> i & 1) {
      const int next = std::min(rank - (sparseDims - i) + 1 + axesAfterEllipsis, rank);
      for (; full < next; full++) { mb[full] = me[full] = true; gather.push_back(full); }
    } else if (newAxisMask >> i & 1) {
      gather.push_back(-2);
    } else {
      ND4J_REQUIRE(full < rank, "StridedSlice: shape calculation failed");
      db[full] = b[i]; de[full] = e[i]; ds[full] = st[i];
      mb[full] = beginMask >> i & 1; me[full] = endMask >> i & 1;
      if (shrinkMask >> i & 1) { shrink[full] = true; gather.push_back(-1); }
      else gather.push_back(full);
      full++;
    }
  }
  SliceGeometry g;
  g.begin.resize(rank); g.count.resize(rank); g.step = ds;
  for (int d = 0; d < rank; d++) {
    const LongType size = x->sizeAt(d), step = ds[d];
    if (shrink[d]) {
      const LongType at = db[d] < 0 ? db[d] + size : db[d];
      ND4J_REQUIRE(at >= 0 && at < size, "StridedSlice: shape calculation failed");
      g.begin[d] = at; g.count[d] = 1; g.step[d] = 1;
      continue;
    }
    // canonical positions: masked = the far ends for this direction; otherwise wrapped once and clamped to what a walk can reach
    const LongType lo = step > 0 ? 0 : -1, hi = step > 0 ? size : size - 1;
    auto canon = [&](LongType v, bool masked, bool isEnd) {
      if (masked) return step > 0 ? (isEnd ? hi : lo) : (isEnd ? lo : hi);
      if (v < 0) v += size;
      return std::max(lo, std::min(hi, v));
    };
    const LongType from = canon(db[d], mb[d], false), to = canon(de[d], me[d], true);
    LongType span = to - from;
    if ((step > 0 && span < 0) || (step < 0 && span > 0)) span = 0;
    const LongType astep = step < 0 ? -step : step, aspan = span < 0 ? -span : span;
    g.begin[d] = from; g.count[d] = (aspan + astep - 1) / astep;
  }
  for (int idx : gather) {
    if (idx == -1) continue;
    g.outShape.push_back(idx == -2 ? 1 : g.count[idx]);
  }
  for (int d = 0; d < rank; d++) if (g.count[d] == 0) g.empty = true;
  return g;
}
static void stridedSliceExec(Context& c) {
  NDArray* x = c.input(0); NDArray* z = c.output(0);
  if (z->isEmpty() || z->lengthOf() == 0) return;
  SliceGeometry g = sliceGeometry(c);
  ND4J_REQUIRE(!g.empty && g.outShape == shapeOf(z), "StridedSlice: output shape " + shapeStr(z) + " does not match the slice");
  LongType offset = 0;
  std::vector<LongType> st(x->rankOf());
  for (int d = 0; d < x->rankOf(); d++) { offset += g.begin[d] * x->strideAt(d); st[d] = g.step[d] * x->strideAt(d); }
  assignEnumerated(z, x, offset, g.count, st, 'c', "StridedSlice");
}
static std::vector<std::vector<LongType>> stridedSliceShapeFn(Context& c) {
  NDArray* x = c.input(0);
  SliceGeometry g = sliceGeometry(c);
  if (g.empty || x->isEmpty()) {
    bool hasZero = false;
    for (auto v : g.outShape) hasZero |= v == 0;
    if (!hasZero) return {makeShapeInfo(x->dataType(), 'c', {}, nullptr, ARRAY_EMPTY)};
    return {makeShapeInfo(x->dataType(), 'c', g.outShape, nullptr, ARRAY_EMPTY)};
  }
  if (g.outShape.empty()) return {scalarShapeInfo(x->dataType())};
  return {makeShapeInfo(x->dataType(), 'c', g.outShape)};
}

// ---- gradient ops ---------------------------------------------------------------------------------------------------------
// softmax_bp (generic/nn/softmax.cpp:53-95): inputs [input, gradO, softmaxedOut], IArg0 = dim (default last);
// gradI = softmaxedOut * (gradO - sum_dim(softmaxedOut * gradO)).  The forward input only supplies the rank.
static void softmaxBpExec(Context& c) {
  ND4J_REQUIRE(c.width() >= 3, "SOFTMAX_BP OP: input, gradO and the softmax output are required");
  NDArray* x = c.input(0);
  NDArray* g = c.input(1);
  NDArray* sm = c.input(2);
  NDArray* z = c.output(0);
  const int rank = x->rankOf();
  int dim = (int)iArg(c, 0, rank - 1);
  ND4J_REQUIRE(dim < rank || rank == 0, "SOFTMAX_BP OP: the value of input integer parameter (dimension) must be less than input array rank " + std::to_string(rank) + ", but got dimension = " + std::to_string(dim) + " instead !");
  if (dim < 0) dim += rank;
  ND4J_REQUIRE(rank == 0 || dim >= 0, "SOFTMAX_BP OP: dimension out of range");
  const DataType dt = z->dataType();
  ND4J_REQUIRE(isFloatType(dt) && g->dataType() == dt && sm->dataType() == dt, "SOFTMAX_BP OP: gradO, the softmax output and gradI must share a floating point type");
  ND4J_REQUIRE(shapeOf(g) == shapeOf(x) && shapeOf(sm) == shapeOf(x) && shapeOf(z) == shapeOf(x), "SOFTMAX_BP OP: all arrays must have the input's shape");
  if (x->isEmpty()) return;
  prepareSpecialUse({z}, {g, sm});
  if (rank == 0) {
    fillValue(z, 0.0);   // a single probability of 1: s * (g - s * g) = 0
  } else {
    RowPlan pg = buildRowPlan(g->shapeInfo(), z->shapeInfo(), dim);
    RowPlan ps = buildRowPlan(sm->shapeInfo(), z->shapeInfo(), dim);
    launchSoftmaxBp(stream(), dt, g->specialBuffer(), sm->specialBuffer(), z->specialBuffer(), pg, ps);
  }
  registerSpecialUse({z}, {g, sm});
}

// standardize (generic/transforms/standardize.cpp:34-78): axes from IArgs or from a second input
static std::vector<LongType> standardizeAxes(Context& c, int axesInput, const char* opName) {
  std::vector<LongType> axes;
  if (axesInput >= 0) axes = hostIndexVector(c.input(axesInput), opName);
  else axes = c.iArgs;
  ND4J_REQUIRE(!axes.empty(), "STANDARDIZE OP: axis has to be non-empty");
  return axes;
}
static void standardizeExec(Context& c) {
  layerNormImpl(c, c.input(0), nullptr, nullptr, c.output(0), standardizeAxes(c, c.width() > 1 ? 1 : -1, "STANDARDIZE OP"), false, "STANDARDIZE OP");
}

// standardize_bp (standardize.cpp:84-154): inputs [input, eps] or [input, axes, eps].  gain (layer_norm_bp only)
// multiplies eps along dimC before the gradient is formed.
static void standardizeBpImpl(NDArray* x, NDArray* eps, NDArray* gain, int dimC, NDArray* z, const std::vector<LongType>& axesIn, const char* opName) {
  const int rank = x->rankOf();
  auto axes = normalizeDims(rank, axesIn.data(), (LongType)axesIn.size(), opName);
  const DataType dt = z->dataType();
  ND4J_REQUIRE(isFloatType(dt) && x->dataType() == dt && eps->dataType() == dt, std::string(opName) + ": nd4j-hip requires input, eps and output to share a floating point type");
  ND4J_REQUIRE(shapeOf(eps) == shapeOf(x) && shapeOf(z) == shapeOf(x), std::string(opName) + ": eps and the output must have the input's shape");
  if (x->isEmpty()) return;
  LnGenericPlan px = lnGenericPlan(x, z, axes, dimC);
  LnGenericPlan pe = lnGenericPlan(eps, z, axes, dimC);
  launchStandardizeBp(stream(), dt, x->specialBuffer(), eps->specialBuffer(), gain ? gain->specialBuffer() : nullptr, z->specialBuffer(), px, pe);
}
static void standardizeBpExec(Context& c) {
  ND4J_REQUIRE(c.width() >= 2, "STANDARDIZE_BP OP: input and eps are required");
  NDArray* x = c.input(0);
  NDArray* eps = c.width() == 3 ? c.input(2) : c.input(1);
  NDArray* z = c.output(0);
  auto axes = standardizeAxes(c, c.width() == 3 ? 1 : -1, "STANDARDIZE_BP OP");
  prepareSpecialUse({z}, {x, eps});
  standardizeBpImpl(x, eps, nullptr, -1, z, axes, "STANDARDIZE_BP OP");
  registerSpecialUse({z}, {x, eps});
}

// layer_norm_bp (generic/nn/layer_norm.cpp:85-157): inputs [input, gain, bias?, eps]; outputs [dLdx, dLdg, dLdb?];
// IArgs = axes, BArg0 = channelsFirst (default true).
//   dLdb = sum of eps over every dim but the channel one
//   dLdg = sum of standardize(input) * eps over the same dims (a fused two-operand reduction of a temporary that holds
//          the standardised input in the array type, as the reference's does)
//   dLdx = standardize_bp(input, eps * gain)
static void layerNormBpExec(Context& c) {
  ND4J_REQUIRE(c.width() >= 3, "LAYER_NORM_BP OP: input, gain and eps arrays are required");
  NDArray* x = c.input(0);
  NDArray* gain = c.input(1);
  NDArray* bias = c.width() == 4 ? c.input(2) : nullptr;
  NDArray* eps = c.width() == 4 ? c.input(3) : c.input(2);
  NDArray* dLdx = c.output(0);
  NDArray* dLdg = c.output(1);
  NDArray* dLdb = c.width() == 4 ? c.output(2) : nullptr;
  const int rank = x->rankOf();
  const bool channelsFirst = bArg(c, 0, true);
  const int dimC = channelsFirst ? 1 : rank - 1;
  ND4J_REQUIRE(dimC < rank, "LAYER_NORM_BP OP: input rank too small for the channel axis");
  ND4J_REQUIRE(gain->rankOf() == 1 && gain->sizeAt(0) == x->sizeAt(dimC),
               "LAYER_NORM_BP OP: wrong shape of gain array, expected is {" + std::to_string(x->sizeAt(dimC)) + "}, but got " + shapeStr(gain) + " instead !");
  if (bias) ND4J_REQUIRE(bias->rankOf() == 1 && bias->sizeAt(0) == x->sizeAt(dimC),
                         "LAYER_NORM_BP OP: wrong shape of bias array, expected is {" + std::to_string(x->sizeAt(dimC)) + "}, but got " + shapeStr(bias) + " instead !");
  const DataType dt = x->dataType();
  ND4J_REQUIRE(isFloatType(dt) && gain->dataType() == dt && eps->dataType() == dt && dLdx->dataType() == dt && dLdg->dataType() == dt && (!dLdb || dLdb->dataType() == dt),
               "LAYER_NORM_BP OP: nd4j-hip requires all arrays to share one floating point type");
  ND4J_REQUIRE(gain->strideAt(0) == 1, "LAYER_NORM_BP OP: gain must be dense");
  ND4J_REQUIRE(dLdg->lengthOf() == gain->lengthOf() && (!dLdb || dLdb->lengthOf() == gain->lengthOf()), "LAYER_NORM_BP OP: wrong length of a parameter gradient");
  ND4J_REQUIRE(!c.iArgs.empty(), "STANDARDIZE OP: axis has to be non-empty");
  if (x->isEmpty()) return;
  std::vector<NDArray*> writes = {dLdx, dLdg}, reads = {x, gain, eps};
  if (dLdb) writes.push_back(dLdb);
  prepareSpecialUse(writes, reads);
  auto lc = LaunchContext::defaultContext();
  std::vector<LongType> others;
  for (int d = 0; d < rank; d++) if (d != dimC) others.push_back(d);
  // a rank-1 descriptor of the parameter gradients lines up with the one kept dim
  if (dLdb) {
    ReducePlan p = buildReducePlan(eps->shapeInfo(), dLdb->shapeInfo(), others, false);
    launchReduce(lc->execStream, R_SUM, dt, dt, eps->specialBuffer(), dLdb->specialBuffer(), p, lc->reductionBuffer, LaunchContext::REDUCTION_BYTES);
  }
  NDArray standardized;
  standardized.si = makeShapeInfo(dt, 'c', shapeOf(x));
  standardized.buf = std::make_shared<DataBuffer>((void*)nullptr, (void*)nullptr, (size_t)x->lengthOf() * sizeOf(dt), dt);
  standardized.buf->allocateSpecial();
  {
    Context sub;
    layerNormImpl(sub, x, nullptr, nullptr, &standardized, c.iArgs, false, "LAYER_NORM_BP OP");
  }
  {
    ReducePlan p = buildReducePlan(standardized.shapeInfo(), dLdg->shapeInfo(), others, false);
    ReducePlan pe = buildReducePlan(eps->shapeInfo(), dLdg->shapeInfo(), others, false);
    launchReduceMisc(lc->execStream, M3_DOT, dt, dt, standardized.specialBuffer(), dLdg->specialBuffer(), p, false, lc->reductionBuffer,
                     LaunchContext::REDUCTION_BYTES, eps->specialBuffer(), dt, &pe);
  }
  standardizeBpImpl(x, eps, gain, dimC, dLdx, c.iArgs, "LAYER_NORM_BP OP");
  HIP_CHECK(hipStreamSynchronize(stream()));   // the temporary is released on return
  registerSpecialUse(writes, reads);
}
static std::vector<std::vector<LongType>> layerNormBpShapeFn(Context& c) {
  auto like = [](NDArray* a) { return makeShapeInfo(a->dataType(), a->ordering(), shapeOf(a)); };
  if (c.width() > 3) return {like(c.input(0)), like(c.input(1)), like(c.input(2))};
  return {like(c.input(0)), like(c.input(1))};
}

// matmul_bp (generic/blas/matmul.cpp:239-332): inputs [x, y, eps], outputs [dLdx, dLdy]; the two gradients are matmuls
// of eps with the other operand under permuted transpose flags.  The scalar-eps branches of the reference (sums of
// the operands times eps) are not implemented.
static void matmulBpExec(Context& c) {
  ND4J_REQUIRE(c.width() >= 3, "MATMUL_BP OP: x, y and eps are required");
  ND4J_REQUIRE(c.outputs.size() >= 2 && c.outputs[1] != nullptr, "MATMUL_BP OP: two output arrays are required");
  NDArray* x = c.input(0);
  NDArray* y = c.input(1);
  NDArray* eps = c.input(2);
  ND4J_REQUIRE(eps->rankOf() != 0, "MATMUL_BP OP: a scalar eps is not implemented in nd4j-hip");
  const LongType transX = iArg(c, 0, 0) ? 1 : 0, transY = iArg(c, 1, 0) ? 1 : 0, transZ = iArg(c, 2, 0) ? 1 : 0;
  Context dx;
  dx.inputs = {eps, y}; dx.outputs = {c.output(0)}; dx.tArgs = {tArg(c, 0, 1.0), tArg(c, 1, 0.0)}; dx.iArgs = {transZ, 1 - transY, transX};
  matmulExec(dx);
  Context dy;
  dy.inputs = {x, eps}; dy.outputs = {c.output(1)}; dy.tArgs = dx.tArgs; dy.iArgs = {1 - transX, transZ, transY};
  matmulExec(dy);
}
static std::vector<std::vector<LongType>> matmulBpShapeFn(Context& c) {
  auto like = [](NDArray* a) { return makeShapeInfo(a->dataType(), a->ordering(), shapeOf(a)); };
  return {like(c.input(0)), like(c.input(1))};
}

// ---- registry ---------------------------------------------------------------------------------------------------------------
static std::map<LongType, OpDescriptor>& byHash() {
  static std::map<LongType, OpDescriptor> m;
  return m;
}
static std::map<std::string, LongType>& byName() {
  static std::map<std::string, LongType> m;
  return m;
}
static void reg(const std::string& name, int nIn, int nOut, bool inplace, int nT, int nI, std::function<void(Context&)> exec,
                std::function<std::vector<std::vector<LongType>>(Context&)> shapeFn) {
  OpDescriptor d{name, opHash(name), nIn, nOut, inplace, nT, nI, std::move(exec), std::move(shapeFn)};
  byName()[name] = d.hash;
  byHash()[d.hash] = std::move(d);
}
static void ensureRegistered() {
  static std::once_flag once;
  std::call_once(once, [] {
    // arities as declared by the reference's *_OP_IMPL macros
    for (const char* alias : {"matmul", "mMul", "mmul", "gemm", "gemv", "dot"}) reg(alias, 2, 1, false, 0, -2, matmulExec, matmulShapeFn);
    reg("xw_plus_b", 3, 1, false, 0, 0, xwPlusBExec, xwPlusBShapeFn);
    reg("softmax", 1, 1, true, 0, 0, softmaxExec, sameAsInputShapeFn);
    reg("log_softmax", 1, 1, true, 0, 0, logSoftmaxExec, sameAsInputShapeFn);
    reg("top_k", 1, 2, false, 0, -1, topKExec, topKShapeFn);
    reg("layer_norm", 2, 1, false, 0, -1, layerNormExec, sameAsInputShapeFn);
    reg("dot_product_attention_v2", -2, -1, false, -2, -2, attentionExec, attentionShapeFn);
    reg("argmax", 1, 1, false, 0, -2, [](Context& c) { argExec(c, 0, "ArgMax"); }, argShapeFn);
    reg("argmin", 1, 1, false, 0, -2, [](Context& c) { argExec(c, 1, "ArgMin"); }, argShapeFn);
    reg("gather", 1, 1, false, 0, -2, gatherExec, gatherShapeFn);
    reg("concat", -1, 1, false, 0, 0, concatExec, concatShapeFn);
    reg("add", 2, 1, true, 0, 0, [](Context& c) { broadcastableExec(c, P_ADD, "ADD OP"); }, broadcastableShapeFn);
    reg("subtract", 2, 1, true, 0, 0, [](Context& c) { broadcastableExec(c, P_SUB, "SUBTRACT OP"); }, broadcastableShapeFn);
    reg("multiply", 2, 1, true, 0, 0, [](Context& c) { broadcastableExec(c, P_MUL, "MULTIPLY OP"); }, broadcastableShapeFn);
    reg("divide", 2, 1, true, 0, 0, [](Context& c) { broadcastableExec(c, P_DIV, "DIVIDE OP"); }, broadcastableShapeFn);
    {
      // the other members of generic/broadcastable/: each applies one legacy pairwise functor under broadcasting
      struct B { const char* name; PairwiseKind k; };
      for (const B& b : {B{"maximum", P_MAX}, B{"minimum", P_MIN}, B{"Pow", P_POW}, B{"realdiv", P_DIV}, B{"reversedivide", P_RDIV},
                         B{"reversesubtract", P_RSUB}, B{"squaredsubtract", P_SQSUB}, B{"floordiv", P_FLOOR_DIV}, B{"floormod", P_FLOOR_MOD},
                         B{"mod", P_MOD}, B{"reversemod", P_REVERSE_MOD}, B{"truncatediv", P_TRUNCATE_DIV}, B{"divide_no_nan", P_DIVIDE_NO_NAN},
                         B{"tf_atan2", P_ATAN2}, B{"assign", P_COPY}}) {
        const PairwiseKind k = b.k; const char* name = b.name;
        reg(b.name, 2, 1, true, 0, 0, [k, name](Context& c) { broadcastableExec(c, k, name); }, broadcastableShapeFn);
      }
    }
    reg("permute", 1, 1, true, 0, -2, [](Context& c) { permuteExec(c, "PERMUTE OP"); }, [](Context& c) { return permuteShapeFn(c, "PERMUTE OP"); });
    reg("transpose", 1, 1, false, 0, 0, [](Context& c) { permuteExec(c, "TRANSPOSE OP"); }, [](Context& c) { return permuteShapeFn(c, "TRANSPOSE OP"); });
    reg("reshape", 1, 1, false, 0, -2, reshapeExec, reshapeShapeFn);
    reg("squeeze", 1, 1, false, 0, -2, [](Context& c) { sameDataExec(c, "squeeze"); }, squeezeShapeFn);
    reg("expand_dims", 1, 1, false, 0, -2, [](Context& c) { sameDataExec(c, "ExpandDims"); }, expandDimsShapeFn);
    reg("split", 1, -1, false, 0, 1, splitExec, splitShapeFn);
    {
      struct R { const char* name; ReduceKind k; const char* label; };
      for (const R& r : {R{"reduce_sum", R_SUM, "REDUCE_SUM OP"}, R{"reduce_max", R_MAX, "REDUCE_MAX OP"}, R{"reduce_min", R_MIN, "REDUCE_MIN OP"},
                         R{"reduce_prod", R_PROD, "REDUCE_PROD OP"}, R{"reduce_mean", R_MEAN, "REDUCE_MEAN OP"}, R{"reduce_norm1", R_NORM1, "REDUCE_NORM1 OP"},
                         R{"reduce_norm2", R_NORM2, "REDUCE_NORM2 OP"}, R{"reduce_norm_max", R_NORMMAX, "REDUCE_NORM_MAX OP"},
                         R{"reduce_sqnorm", R_SQNORM, "REDUCE_SQNORM OP"}}) {
        const ReduceKind k = r.k; const char* label = r.label;
        reg(r.name, -1, 1, false, 0, 0, [k, label](Context& c) { reduceCustomExec(c, k, label); }, [label](Context& c) { return reduceCustomShapeFn(c, label); });
      }
      reg("reduce_variance", -1, 1, false, 0, 0, [](Context& c) { reduceStatsExec(c, M_VARIANCE, "REDUCE_VARIANCE OP"); }, [](Context& c) { return reduceCustomShapeFn(c, "REDUCE_VARIANCE OP"); });
      reg("reduce_stdev", -1, 1, false, 0, 0, [](Context& c) { reduceStatsExec(c, M_STDDEV, "REDUCE_STDEV OP"); }, [](Context& c) { return reduceCustomShapeFn(c, "REDUCE_STDEV OP"); });
    }
    {
      struct U { const char* name; UnaryKind k; };
      for (const U& u : {U{"tanh", U_TANH}, U{"sigmoid", U_SIGMOID}, U{"softplus", U_SOFTPLUS}, U{"softsign", U_SOFTSIGN}, U{"cube", U_CUBE},
                         U{"hardsigmoid", U_HARD_SIGMOID}, U{"hardtanh", U_HARD_TANH}, U{"rationaltanh", U_RATIONAL_TANH},
                         U{"rectifiedtanh", U_RECTIFIED_TANH}, U{"selu", U_SELU}, U{"identity", U_IDENTITY}}) {
        const UnaryKind k = u.k; const char* name = u.name;
        reg(u.name, 1, 1, true, 0, 0, [k, name](Context& c) { activationExec(c, k, name); }, sameAsInputShapeFn);
      }
      reg("relu", 1, 1, true, 1, 0, [](Context& c) { scalarActivationExec(c, P_RELU, 0.0, "relu"); }, sameAsInputShapeFn);
      reg("relu6", 1, 1, true, 1, 0, [](Context& c) { scalarActivationExec(c, P_RELU6, 0.0, "relu6"); }, sameAsInputShapeFn);
      reg("lrelu", 1, 1, true, -2, 0, [](Context& c) { scalarActivationExec(c, P_LEAKY_RELU, 0.01f, "lrelu"); }, sameAsInputShapeFn);
      reg("elu", 1, 1, true, -2, 0, [](Context& c) { scalarActivationExec(c, P_ELU, 1.0, "elu"); }, sameAsInputShapeFn);
    }
    for (const char* alias : {"clipbyvalue", "ClipByValue"}) reg(alias, -2, 1, true, -2, 0, clipByValueExec, sameAsInputShapeFn);
    reg("softmax_bp", 3, 1, true, 0, 0, softmaxBpExec, sameAsInputShapeFn);
    reg("standardize", 1, 1, true, 0, -2, standardizeExec, sameAsInputShapeFn);
    reg("standardize_bp", 2, 1, false, 0, -2, standardizeBpExec, sameAsInputShapeFn);
    reg("layer_norm_bp", 3, -1, false, 0, -1, layerNormBpExec, layerNormBpShapeFn);
    reg("matmul_bp", 3, 2, false, 0, -2, matmulBpExec, matmulBpShapeFn);
    {
      struct { const char* name; PairwiseKind kind; } cmp[] = {{"equals", P_EQ}, {"equal", P_EQ}, {"not_equals", P_NE}, {"greater", P_GT},
                                                               {"greater_equal", P_GE}, {"less", P_LT}, {"less_equal", P_LE}};
      for (auto& e : cmp) {
        const PairwiseKind kind = e.kind; const char* name = e.name;
        reg(name, 2, 1, true, 0, 0, [kind, name](Context& c) { comparisonExec(c, kind, name); }, comparisonShapeFn);
      }
    }
    for (const char* alias : {"zeros_as", "zeroslike", "zeros_like"}) reg(alias, 1, 1, false, 0, 0, [](Context& c) { fillAsExec(c, 0.0, "zeros_as"); }, fillAsShapeFn);
    reg("ones_as", 1, 1, false, 0, 0, [](Context& c) { fillAsExec(c, 1.0, "ones_as"); }, fillAsShapeFn);
    reg("tile", 1, 1, false, 0, -2, tileExec, tileShapeFn);
    reg("slice", 1, 1, false, 0, -2, sliceExec, sliceShapeFn);
    for (const char* alias : {"biasadd", "bias_add"}) reg(alias, 2, 1, true, 0, 0, biasAddExec, biasAddShapeFn);
    for (const char* alias : {"cast", "Cast"}) reg(alias, 1, 1, false, 0, -2, castExec, castShapeFn);
    for (const char* alias : {"stack", "pack", "Pack"}) reg(alias, -1, 1, false, 0, 0, stackExec, stackShapeFn);
    for (const char* alias : {"unstack", "unpack"}) reg(alias, 1, -1, false, 0, 1, unstackExec, unstackShapeFn);
    for (const char* alias : {"strided_slice", "stridedslice"}) reg(alias, 1, 1, false, 0, 5, stridedSliceExec, stridedSliceShapeFn);
  });
}
const OpDescriptor* findOp(LongType hash) {
  ensureRegistered();
  auto it = byHash().find(hash);
  return it == byHash().end() ? nullptr : &it->second;
}
const OpDescriptor* findOpByName(const std::string& name) {
  ensureRegistered();
  auto it = byName().find(name);
  return it == byName().end() ? nullptr : findOp(it->second);
}
const char* allCustomOps() {
  ensureRegistered();
  static std::string list;
  static std::once_flag once;
  std::call_once(once, [] {
    for (auto& kv : byName()) {
      const OpDescriptor& d = byHash()[kv.second];
      list += d.name + ":" + std::to_string(d.hash) + ":" + std::to_string(d.nIn) + ":" + std::to_string(d.nOut) + ":" +
              std::to_string((int)d.inplace) + ":" + std::to_string(d.nT) + ":" + std::to_string(d.nI) + ":;";
    }
  });
  return list.c_str();
}

void executeOp(const OpDescriptor& op, Context& ctx) {
  // DeclarableOp::execute validations (ops/declarable/impl/DeclarableOp.cpp:866-919): arity and null checks
  if (op.nIn > 0) ND4J_REQUIRE(ctx.width() >= op.nIn, "Op [" + op.name + "] expects at least " + std::to_string(op.nIn) + " input arrays, got " + std::to_string(ctx.width()));
  for (int i = 0; i < ctx.width(); i++) ND4J_REQUIRE(ctx.inputs[i] != nullptr, "Op [" + op.name + "]: input array " + std::to_string(i) + " is null");
  ND4J_REQUIRE(!ctx.outputs.empty() && ctx.outputs[0] != nullptr, "Op [" + op.name + "]: output array 0 is missing (outputs must be supplied; use calculateOutputShapes2 to size them)");
  op.exec(ctx);
}


// ---- merging of recorded op sequences -----------------------------------------------------------------------------------
// the two handles name the same elements: same buffer, offset, shape, strides and type
static bool sameView(const NDArray* a, const NDArray* b) {
  if (a == b) return true;
  if (!a || !b || a->buf.get() != b->buf.get() || a->bufOffsetBytes != b->bufOffsetBytes || a->offset != b->offset) return false;
  if (a->rankOf() != b->rankOf() || a->dataType() != b->dataType()) return false;
  for (int d = 0; d < a->rankOf(); d++) if (a->sizeAt(d) != b->sizeAt(d) || (a->sizeAt(d) != 1 && a->strideAt(d) != b->strideAt(d))) return false;
  return true;
}
// a view seen as [rows, cols] with a unit column stride and one row stride: all dims but the last fold into the rows
static bool asRows(const NDArray* a, LongType& rows, LongType& cols, LongType& rowStride) {
  const int r = a->rankOf();
  if (r < 1 || a->isEmpty()) return false;
  cols = a->sizeAt(r - 1);
  if (cols != 1 && a->strideAt(r - 1) != 1) return false;
  rows = 1; rowStride = 0;
  LongType expect = -1;
  for (int d = r - 2; d >= 0; d--) {
    const LongType n = a->sizeAt(d);
    if (n == 1) continue;
    if (expect < 0) rowStride = a->strideAt(d);
    else if (a->strideAt(d) != expect) return false;
    expect = a->strideAt(d) * n;
    rows *= n;
  }
  if (rows == 1) rowStride = cols;
  return true;
}
static bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

// layer_norm over the last axis with gain and bias, as the row kernel runs it
static bool isRowLayerNorm(const RecordedOp& r) {
  if (r.kind != RecordedOp::CUSTOM || r.op->name != "layer_norm" || r.ctx.inputs.size() != 3 || r.ctx.outputs.empty()) return false;
  const NDArray* x = r.ctx.inputs[0];
  if (!x || !r.ctx.inputs[1] || !r.ctx.inputs[2] || !r.ctx.outputs[0] || x->rankOf() < 1) return false;
  if (bArg(r.ctx, 0, true)) return false;                            // gain / bias along the last axis
  if (r.ctx.iArgs.size() != 1) return false;
  const LongType ax = r.ctx.iArgs[0] < 0 ? r.ctx.iArgs[0] + x->rankOf() : r.ctx.iArgs[0];
  return ax == x->rankOf() - 1;
}

static void runRecorded(RecordedOp* p) {
  if (p->kind == RecordedOp::CUSTOM) executeOp(*p->op, p->ctx);
  else p->run(*p);
}
// z = x + y (pairwise Add, all of one float type), then ln = layer_norm(z): one kernel
static bool tryAddLayerNorm(const RecordedOp& add, const RecordedOp& ln) {
  NDArray *x = add.x, *y = add.y, *z = add.z;
  NDArray *lx = ln.ctx.inputs[0], *g = ln.ctx.inputs[1], *b = ln.ctx.inputs[2], *lz = ln.ctx.outputs[0];
  const DataType dt = z->dataType();
  if (!isFloatType(dt) || dt == DOUBLE || x->dataType() != dt || y->dataType() != dt || lz->dataType() != dt || g->dataType() != dt || b->dataType() != dt) return false;
  LongType rx, cx, sx, ry, cy, sy, rz, cz, sz, rl, cl, sl;
  if (!asRows(x, rx, cx, sx) || !asRows(y, ry, cy, sy) || !asRows(z, rz, cz, sz) || !asRows(lz, rl, cl, sl)) return false;
  if (rx != rz || ry != rz || rl != rz || cx != cz || cy != cz || cl != cz) return false;
  if (g->lengthOf() != cz || b->lengthOf() != cz || (g->rankOf() == 1 && g->strideAt(0) != 1 && cz > 1) || (b->rankOf() == 1 && b->strideAt(0) != 1 && cz > 1)) return false;
  // the normalised output must not overlap what the merged kernel still reads
  if (lz->buf.get() == x->buf.get() || lz->buf.get() == y->buf.get() || lz->buf.get() == z->buf.get()) return false;
  if (y->buf.get() == z->buf.get() && !sameView(y, z)) return false;
  if (x->buf.get() == z->buf.get() && !sameView(x, z)) return false;
  std::vector<NDArray*> writes = {z, lz}, reads = {x, y, g, b};
  prepareSpecialUse(writes, reads);
  const bool ok = launchAddLayerNormRows(stream(), dt, x->specialBuffer(), y->specialBuffer(), z->specialBuffer(), g->specialBuffer(), b->specialBuffer(),
                                         lz->specialBuffer(), rz, cz, sx, sy, sz, sl, 1e-5f);
  registerSpecialUse(writes, reads);
  return ok;
}

}  // namespace ops

void RecordedOp::adopt() {
  std::vector<std::pair<NDArray*, NDArray*>> seen;   // one copy per handle: an op called in place keeps input == output
  auto own = [&](NDArray*& a) {
    if (!a) return;
    for (auto& s : seen) if (s.first == a) { a = s.second; return; }
    owned.push_back(std::make_shared<NDArray>(*a));
    seen.emplace_back(a, owned.back().get());
    a = owned.back().get();
  };
  own(x); own(y); own(z);
  for (NDArray*& a : ctx.inputs) own(a);
  for (NDArray*& a : ctx.outputs) own(a);
}

int& fusedAppliedCounter() { static int n = 0; return n; }

std::vector<std::function<void()>> fuseRecordedOps(std::vector<RecordedOp>& rec, int& nFused) {
  using namespace ops;
  std::vector<std::function<void()>> plan;
  nFused = 0;
  const size_t n = rec.size();
  // is rec[li] a layer_norm that the xw_plus_b behind it can run as its prologue (products of one row, and of 5 to 32 rows
  // of 320 to 768 values, the lengths the few-row product kernel normalises)?
  auto lnPrologueAt = [&](size_t li, LnPrologue& out) {
    if (li + 1 >= n) return false;
    RecordedOp& r = rec[li];
    RecordedOp& x = rec[li + 1];
    if (!isRowLayerNorm(r) || x.kind != RecordedOp::CUSTOM || x.op->name != "xw_plus_b" || x.ctx.inputs.size() < 3 || !x.ctx.inputs[0] ||
        !sameView(x.ctx.inputs[0], r.ctx.outputs[0])) return false;
    NDArray *lx = r.ctx.inputs[0], *lg = r.ctx.inputs[1], *lb = r.ctx.inputs[2], *lo = r.ctx.outputs[0];
    LongType rr, cc, ss, r2, c2, s2;
    const DataType dt = lx->dataType();
    const bool ok = (dt == HALF || dt == BFLOAT16) && lg->dataType() == dt && lb->dataType() == dt && lo->dataType() == dt && asRows(lx, rr, cc, ss) &&
                    (rr == 1 || (rr >= 5 && rr <= 32 && cc >= 320 && cc <= 768 && cc % 64 == 0)) && asRows(lo, r2, c2, s2) && r2 == rr && c2 == cc && lg->lengthOf() == cc && lb->lengthOf() == cc &&
                    lo->buf.get() != lx->buf.get() && iArg(x.ctx, 0, 0) != 1;
    if (!ok) return false;
    out = LnPrologue{lx, lg, lb, lo, rr, ss, s2};
    return true;
  };
  // is rec[li] an attention (output only) whose output row -- one query, the heads side by side -- is the input row of the
  // xw_plus_b behind it?  Then, when the attention cuts its key range up, that product merges the parts on its way in.
  auto attnMergeAt = [&](size_t li) {
    if (li + 1 >= n) return false;
    RecordedOp& r = rec[li];
    RecordedOp& x = rec[li + 1];
    if (r.kind != RecordedOp::CUSTOM || r.op->name != "dot_product_attention_v2" || r.ctx.outputs.empty() || !r.ctx.outputs[0]) return false;
    for (size_t o = 1; o < r.ctx.outputs.size(); o++) if (r.ctx.outputs[o]) return false;
    if (x.kind != RecordedOp::CUSTOM || x.op->name != "xw_plus_b" || x.ctx.inputs.size() < 3 || !x.ctx.inputs[0] || iArg(x.ctx, 0, 0) == 1) return false;
    NDArray *o = r.ctx.outputs[0], *in = x.ctx.inputs[0];
    if (o->buf.get() != in->buf.get() || o->offset != in->offset || o->dataType() != in->dataType() || o->lengthOf() != in->lengthOf()) return false;
    LongType rr, cc, ss;
    if (!asRows(in, rr, cc, ss) || rr != 1 || o->rankOf() < 2) return false;
    // the output's elements in (head, value) order must be the row's elements in order: one query, unit value stride, heads D apart
    const int rank = o->rankOf();
    const LongType D = o->sizeAt(rank - 1);
    if (o->sizeAt(rank - 2) != 1 || (D > 1 && o->strideAt(rank - 1) != 1)) return false;
    LongType heads = 1;
    for (int d = 0; d < rank - 2; d++) {
      if (o->sizeAt(d) == 1) continue;
      if (d != rank - 3 || o->strideAt(d) != D) return false;
      heads = o->sizeAt(d);
    }
    return heads * D == cc;
  };
  for (size_t i = 0; i < n;) {
    RecordedOp& r = rec[i];
    // pairwise Add whose result the next op layer-normalises
    if (r.kind == RecordedOp::PAIRWISE && r.opNum == 0 && i + 1 < n && isRowLayerNorm(rec[i + 1]) && sameView(r.z, rec[i + 1].ctx.inputs[0])) {
      RecordedOp* a = &r;
      RecordedOp* l = &rec[i + 1];
      plan.push_back([a, l] { if (tryAddLayerNorm(*a, *l)) fusedAppliedCounter() += 1; else { runRecorded(a); runRecorded(l); } });
      nFused += 1;
      i += 2;
      continue;
    }
    // xw_plus_b, with the ops around it that its kernel can take in: in front a layer_norm whose output row is the
    // product's input (one-row products normalise the row on the way in), behind it ops on the result that the epilogue can
    // write -- the GELU transform of the whole result, assigns of column slices (key / value rows going into their
    // caches), a pairwise Add of the result to another array (the residual connection)
    {
      RecordedOp* lnOp = nullptr;
      RecordedOp* attnOp = nullptr;
      LnPrologue lnPro{};
      size_t xi = i;
      if (lnPrologueAt(i, lnPro)) { lnOp = &r; xi = i + 1; }
      else if (attnMergeAt(i)) { attnOp = &r; xi = i + 1; }
      RecordedOp& xw = rec[xi];
      if (xw.kind == RecordedOp::CUSTOM && xw.op->name == "xw_plus_b" && xw.ctx.outputs.size() >= 1 && xw.ctx.outputs[0] && xw.ctx.inputs.size() >= 3 &&
          xw.ctx.inputs[0] && xw.ctx.inputs[1] && xw.ctx.inputs[2]) {
        NDArray* z = xw.ctx.outputs[0];
        LongType zr = 0, zc = 0, zs = 0;
        const DataType dt = z->dataType();
        const bool zOk = (dt == HALF || dt == BFLOAT16) && asRows(z, zr, zc, zs) && iArg(xw.ctx, 2, 0) != 1;
        GemmEpilogue epi;          // array handles for now; device pointers when the step runs
        std::vector<RecordedOp*> absorbed;
        LnPrologue lnAhead{};
        size_t j = xi + 1;
        while (zOk && j < n) {
          RecordedOp& f = rec[j];
          if (f.kind == RecordedOp::CUSTOM || f.z == nullptr) break;
          bool clash = f.z->buf.get() == z->buf.get();   // an absorbed op writes neither the product's operands nor its result
          for (NDArray* in : xw.ctx.inputs) if (in && in->buf.get() == f.z->buf.get()) clash = true;
          if (lnOp) for (NDArray* in : lnOp->ctx.inputs) if (in && in->buf.get() == f.z->buf.get()) clash = true;
          if (attnOp) for (NDArray* in : attnOp->ctx.inputs) if (in && in->buf.get() == f.z->buf.get()) clash = true;
          if (clash || f.z->dataType() != dt) break;
          LongType fr, fc, fs;
          if (f.kind == RecordedOp::TRANSFORM_STRICT && f.opNum == 53 && epi.act == 0 && sameView(f.x, z) && asRows(f.z, fr, fc, fs) && fr == zr && fc == zc) {
            // the form the separate transform takes on dense, aligned 16-bit arrays of a multiple of 8 elements
            if (!(zs == zc && fs == fc && (zr * zc) % 8 == 0)) break;
            epi.act = 1; epi.actOut = f.z; epi.actRow = fs;
          } else if (f.kind == RecordedOp::TRANSFORM_ANY && epi.nCopy < 2 && f.x->buf.get() == z->buf.get() && f.x->bufOffsetBytes == z->bufOffsetBytes &&
                     f.x->dataType() == dt) {
            LongType sr, sc, ss, dr, dc, ds;
            if (!asRows(f.x, sr, sc, ss) || !asRows(f.z, dr, dc, ds) || sr != zr || dr != zr || dc != sc || (zr > 1 && ss != zs)) break;
            const LongType c0 = f.x->offset - z->offset;
            if (c0 < 0 || c0 + sc > zc) break;
            epi.copy[epi.nCopy].dst = f.z; epi.copy[epi.nCopy].c0 = c0; epi.copy[epi.nCopy].c1 = c0 + sc; epi.copy[epi.nCopy].dstRow = ds;
            epi.nCopy++;
          } else if (f.kind == RecordedOp::PAIRWISE && f.opNum == 0 && epi.resOut == nullptr && (sameView(f.y, z) || sameView(f.x, z)) &&
                     f.x->dataType() == dt && f.y->dataType() == dt &&
                     (zr == 1 || (zr >= 5 && zr <= 32 && j + 1 < n && isRowLayerNorm(rec[j + 1]) && sameView(f.z, rec[j + 1].ctx.inputs[0]) && lnPrologueAt(j + 1, lnAhead)))) {
            // (one-row products, and the few-row ones whose sum goes into a layer_norm that the next product normalises on its
            // way in; otherwise the Add merges with the layer_norm behind it, which measured faster than per-element residual
            // traffic in the tile kernels' epilogues)
            NDArray* other = sameView(f.y, z) ? f.x : f.y;   // the addition commutes bit for bit
            LongType orr, oc, os;
            if (other->buf.get() == z->buf.get() || !asRows(other, orr, oc, os) || !asRows(f.z, fr, fc, fs) || orr != zr || oc != zc || fr != zr || fc != zc) break;
            if (other->buf.get() == f.z->buf.get() && !sameView(other, f.z)) break;
            epi.resIn = other; epi.resInRow = os; epi.resOut = f.z; epi.resOutRow = fs;
          } else {
            break;
          }
          absorbed.push_back(&f);
          j++;
          // nothing may follow an absorbed Add inside this kernel: later ops read its result
          if (f.kind == RecordedOp::PAIRWISE) break;
        }
        if (lnOp || attnOp || !absorbed.empty()) {
          RecordedOp* x = &xw;
          plan.push_back([x, lnOp, attnOp, lnPro, epi, absorbed] {
            GemmEpilogue e = epi;
            NDArray* z = x->ctx.outputs[0];
            std::vector<NDArray*> writes, reads;
            NDArray* actArr = static_cast<NDArray*>(epi.actOut);
            if (e.act) writes.push_back(actArr);
            for (int c = 0; c < e.nCopy; c++) writes.push_back(static_cast<NDArray*>(epi.copy[c].dst));
            if (e.resOut) { writes.push_back(static_cast<NDArray*>(epi.resOut)); reads.push_back(static_cast<NDArray*>(const_cast<void*>(epi.resIn))); }
            z->buf->allocateSpecial();
            prepareSpecialUse(writes, reads);
            if (e.act) e.actOut = actArr->specialBuffer();
            for (int c = 0; c < e.nCopy; c++) e.copy[c].dst = static_cast<NDArray*>(epi.copy[c].dst)->specialBuffer();
            if (e.resOut) { e.resOut = static_cast<NDArray*>(epi.resOut)->specialBuffer(); e.resIn = static_cast<NDArray*>(const_cast<void*>(epi.resIn))->specialBuffer(); }
            // a misaligned GELU operand would send the separate transform down another evaluation path: keep the ops apart then
            const bool epiOk = !absorbed.empty() && !(e.act && (!aligned16(z->specialBuffer()) || !aligned16(e.actOut)));
            const GemmEpilogue* ep = epiOk ? &e : nullptr;
            bool applied = false, done = false;
            if (lnOp) {
              done = xwPlusBImpl(x->ctx, ep, &lnPro);
              applied = done && epiOk;
              if (done) fusedAppliedCounter() += 1; else runRecorded(lnOp);
            }
            if (attnOp) {
              // the attention runs as recorded; where it cuts its key range up it leaves the merge to this product
              AttnMergeRequest req;
              g_attnMergeRequest = &req;
              try { runRecorded(attnOp); } catch (...) { g_attnMergeRequest = nullptr; throw; }
              g_attnMergeRequest = nullptr;
              if (req.deferred) {
                NDArray* ao = attnOp->ctx.outputs[0];
                AttnMergePrologue am{req.desc.partial, req.desc.splits, (int)req.desc.D, ao};
                done = xwPlusBImpl(x->ctx, ep, nullptr, &am);
                applied = done && epiOk;
                if (!done) launchAttentionDecodeMerge(stream(), req.dt, ao->specialBuffer(), req.desc);   // the product declined: merge, then multiply
              }
            }
            if (!done) applied = xwPlusBImpl(x->ctx, ep) && epiOk;
            if (applied) fusedAppliedCounter() += (int)absorbed.size();
            if (applied) registerSpecialUse(writes, reads);
            else for (RecordedOp* f : absorbed) runRecorded(f);
          });
          nFused += (int)absorbed.size() + (lnOp ? 1 : 0);
          i = j;
          continue;
        }
      }
    }
    RecordedOp* p = &r;
    plan.push_back([p] { runRecorded(p); });
    i++;
  }
  return plan;
}

}  // namespace nd4jhip
