#include "plan.h"

#include <algorithm>

namespace nd4jhip {

int collapseDims(int rank, LongType* shp, LongType* const* strides, int nOps) {
  // drop unit dims
  int r = 0;
  for (int d = 0; d < rank; d++) {
    if (shp[d] == 1) continue;
    shp[r] = shp[d];
    for (int o = 0; o < nOps; o++) strides[o][r] = strides[o][d];
    r++;
  }
  if (r == 0) {
    shp[0] = 1;
    for (int o = 0; o < nOps; o++) strides[o][0] = 1;
    return 1;
  }
  // merge dim d+1 into d when stride[d] == shape[d+1] * stride[d+1] for every operand
  int w = 0;
  for (int d = 1; d < r; d++) {
    bool merge = true;
    for (int o = 0; o < nOps; o++)
      if (strides[o][w] != shp[d] * strides[o][d]) merge = false;
    if (merge) {
      shp[w] *= shp[d];
      for (int o = 0; o < nOps; o++) strides[o][w] = strides[o][d];
    } else {
      w++;
      shp[w] = shp[d];
      for (int o = 0; o < nOps; o++) strides[o][w] = strides[o][d];
    }
  }
  return w + 1;
}

DevShape toDevShape(const std::vector<LongType>& shp, const std::vector<LongType>& stride) {
  ND4J_REQUIRE(shp.size() <= (size_t)MAX_DEV_RANK, "array rank (after collapsing) above 8 is not supported on device");
  DevShape s;
  s.rank = (int)shp.size();
  for (int i = 0; i < MAX_DEV_RANK; i++) { s.shape[i] = 1; s.stride[i] = 0; }
  for (int i = 0; i < s.rank; i++) { s.shape[i] = shp[i]; s.stride[i] = stride[i]; }
  return s;
}

static DevShape devShapeOf(const LongType* si) {
  int r = shape::rank(si);
  std::vector<LongType> shp(shape::shapeOf(si), shape::shapeOf(si) + r), st(shape::strideOf(si), shape::strideOf(si) + r);
  // collapse on its own so that high-rank arrays still fit
  std::vector<LongType*> ptr = {st.data()};
  if (r > 0) {
    int nr = collapseDims(r, shp.data(), ptr.data(), 1);
    shp.resize(nr); st.resize(nr);
  }
  return toDevShape(shp, st);
}

static LongType maxOffset(int rank, const LongType* shp, const LongType* st) {
  LongType m = 0;
  for (int d = 0; d < rank; d++) m += (shp[d] - 1) * (st[d] < 0 ? -st[d] : st[d]);
  return m;
}

EwPlan buildEwPlan(const std::vector<const LongType*>& ops) {
  EwPlan p;
  p.nOperands = (int)ops.size();
  ND4J_REQUIRE(p.nOperands >= 2 && p.nOperands <= 3, "elementwise plan takes 2 or 3 operands");
  p.length = shape::length(ops[0]);
  for (auto si : ops) ND4J_REQUIRE(shape::length(si) == p.length, "elementwise op: operands must have equal lengths");
  const int r0 = shape::rank(ops[0]);
  p.sameShape = true;
  for (auto si : ops) {
    if (shape::rank(si) != r0) { p.sameShape = false; break; }
    for (int d = 0; d < r0; d++) if (shape::shapeOf(si)[d] != shape::shapeOf(ops[0])[d]) p.sameShape = false;
  }
  for (int o = 0; o < p.nOperands; o++) p.own[o] = devShapeOf(ops[o]);
  for (int o = p.nOperands; o < 3; o++) p.own[o] = p.own[1];
  p.index32 = p.length < (1LL << 31);
  if (!p.sameShape) {
    // equal lengths, different shapes: if every operand is dense row-major they still iterate alike
    bool allDense = true;
    for (int o = 0; o < p.nOperands; o++) if (!(p.own[o].rank == 1 && p.own[o].stride[0] == 1)) allDense = false;
    if (allDense) {
      p.sameShape = true; p.rank = 1; p.shape[0] = p.length; p.contiguous = true;
      for (int o = 0; o < 3; o++) p.stride[o][0] = 1;
    }
    return p;
  }
  std::vector<LongType> shp(std::max(r0, 1), 1);
  std::vector<std::vector<LongType>> st(p.nOperands, std::vector<LongType>(std::max(r0, 1), 1));
  for (int d = 0; d < r0; d++) shp[d] = shape::shapeOf(ops[0])[d];
  for (int o = 0; o < p.nOperands; o++) for (int d = 0; d < r0; d++) st[o][d] = shape::strideOf(ops[o])[d];
  // same shape everywhere: the result does not depend on the visiting order, so visit the dims in
  // descending order of the output's strides (turns 'f'-ordered operands into unit-stride inner runs)
  if (r0 > 1) {
    std::vector<int> perm(r0);
    for (int d = 0; d < r0; d++) perm[d] = d;
    std::stable_sort(perm.begin(), perm.end(), [&](int a, int b) {
      LongType sa = st[0][a] < 0 ? -st[0][a] : st[0][a], sb = st[0][b] < 0 ? -st[0][b] : st[0][b];
      return sa > sb;
    });
    std::vector<LongType> shp2(r0);
    std::vector<std::vector<LongType>> st2(p.nOperands, std::vector<LongType>(r0));
    for (int d = 0; d < r0; d++) {
      shp2[d] = shp[perm[d]];
      for (int o = 0; o < p.nOperands; o++) st2[o][d] = st[o][perm[d]];
    }
    shp = shp2;
    st = st2;
  }
  std::vector<LongType*> ptr;
  for (auto& v : st) ptr.push_back(v.data());
  int nr = collapseDims(std::max(r0, 1), shp.data(), ptr.data(), p.nOperands);
  if (nr > MAX_DEV_RANK) { p.sameShape = false; return p; }
  p.rank = nr;
  for (int d = 0; d < nr; d++) {
    p.shape[d] = shp[d];
    for (int o = 0; o < p.nOperands; o++) p.stride[o][d] = st[o][d];
    for (int o = p.nOperands; o < 3; o++) p.stride[o][d] = st[1][d];
  }
  p.contiguous = nr == 1;
  for (int o = 0; o < p.nOperands; o++) {
    if (p.stride[o][0] != 1 && nr == 1) p.contiguous = false;
    if (maxOffset(nr, shp.data(), st[o].data()) >= (1LL << 31)) p.index32 = false;
    // negative strides are walked with 64-bit arithmetic
    for (int d = 0; d < nr; d++) if (st[o][d] < 0) p.index32 = false;
  }
  return p;
}

std::vector<LongType> normalizeDims(int rank, const LongType* dims, LongType n, const char* what) {
  std::vector<LongType> out;
  for (LongType i = 0; i < n; i++) {
    LongType d = dims[i];
    if (d == 2147483647LL) continue;  // "all dimensions" marker used by the Java side
    if (d < 0) d += rank;
    ND4J_REQUIRE(d >= 0 && d < rank, std::string(what) + ": dimension out of range");
    if (std::find(out.begin(), out.end(), d) == out.end()) out.push_back(d);
  }
  std::sort(out.begin(), out.end());
  return out;
}

ReducePlan buildReducePlan(const LongType* xsi, const LongType* zsi, const std::vector<LongType>& dims, bool zLinear) {
  ReducePlan p;
  const int r = shape::rank(xsi);
  std::vector<bool> red(std::max(r, 1), false);
  if (dims.empty()) for (int d = 0; d < r; d++) red[d] = true;
  for (auto d : dims) red[d] = true;
  std::vector<LongType> oshape, ostride, ishape, istride;
  for (int d = 0; d < r; d++) {
    if (red[d]) { ishape.push_back(shape::shapeOf(xsi)[d]); istride.push_back(shape::strideOf(xsi)[d]); }
    else { oshape.push_back(shape::shapeOf(xsi)[d]); ostride.push_back(shape::strideOf(xsi)[d]); }
  }
  p.outerLen = 1; for (auto s : oshape) p.outerLen *= s;
  p.innerLen = 1; for (auto s : ishape) p.innerLen *= s;
  ND4J_REQUIRE(shape::length(zsi) == p.outerLen,
               "reduce: output length " + std::to_string(shape::length(zsi)) + " does not match the kept dimensions (" + std::to_string(p.outerLen) + ")");
  // z strides for the kept dims: skip z's unit dims (keepDims) unless the kept dim itself has extent 1
  std::vector<LongType> zstride;
  {
    const int zr = shape::rank(zsi);
    std::vector<LongType> zs, zsh;
    for (int d = 0; d < zr; d++) if (shape::shapeOf(zsi)[d] != 1) { zsh.push_back(shape::shapeOf(zsi)[d]); zs.push_back(shape::strideOf(zsi)[d]); }
    size_t q = 0;
    for (size_t d = 0; d < oshape.size(); d++) {
      if (oshape[d] == 1) { zstride.push_back(0); continue; }
      ND4J_REQUIRE(q < zsh.size() && zsh[q] == oshape[d], "reduce: output shape does not line up with the kept dimensions");
      zstride.push_back(zs[q++]);
    }
  }
  // collapse inner dims on their own; outer dims jointly for x and z
  if (!ishape.empty()) {
    std::vector<LongType*> ptr = {istride.data()};
    int nr = collapseDims((int)ishape.size(), ishape.data(), ptr.data(), 1);
    ishape.resize(nr); istride.resize(nr);
  }
  if (!oshape.empty()) {
    std::vector<LongType*> ptr = {ostride.data(), zstride.data()};
    int nr = collapseDims((int)oshape.size(), oshape.data(), ptr.data(), 2);
    oshape.resize(nr); ostride.resize(nr); zstride.resize(nr);
  }
  p.outer = toDevShape(oshape, ostride);
  p.zOuter = toDevShape(oshape, zstride);
  p.inner = toDevShape(ishape, istride);
  p.zLinear = zLinear;
  p.index32 = shape::length(xsi) < (1LL << 31);
  return p;
}

RowPlan buildRowPlan(const LongType* xsi, const LongType* zsi, int dim) {
  RowPlan p;
  const int r = shape::rank(xsi);
  ND4J_REQUIRE(shape::rank(zsi) == r, "row op: input and output ranks differ");
  for (int d = 0; d < r; d++) ND4J_REQUIRE(shape::shapeOf(xsi)[d] == shape::shapeOf(zsi)[d], "row op: input and output shapes differ");
  if (r == 0) {
    p.rows = 1; p.rowLen = 1; p.xInner = p.zInner = 1;
    p.outerX = toDevShape({}, {}); p.outerZ = toDevShape({}, {});
    return p;
  }
  if (dim < 0) dim += r;
  ND4J_REQUIRE(dim >= 0 && dim < r, "row op: dimension out of range");
  p.rowLen = shape::shapeOf(xsi)[dim];
  p.xInner = shape::strideOf(xsi)[dim];
  p.zInner = shape::strideOf(zsi)[dim];
  std::vector<LongType> oshape, xs, zs;
  for (int d = 0; d < r; d++) {
    if (d == dim) continue;
    oshape.push_back(shape::shapeOf(xsi)[d]); xs.push_back(shape::strideOf(xsi)[d]); zs.push_back(shape::strideOf(zsi)[d]);
  }
  p.rows = 1; for (auto s : oshape) p.rows *= s;
  if (!oshape.empty()) {
    std::vector<LongType*> ptr = {xs.data(), zs.data()};
    int nr = collapseDims((int)oshape.size(), oshape.data(), ptr.data(), 2);
    oshape.resize(nr); xs.resize(nr); zs.resize(nr);
  }
  p.outerX = toDevShape(oshape, xs);
  p.outerZ = toDevShape(oshape, zs);
  p.index32 = shape::length(xsi) < (1LL << 31);
  return p;
}

}  // namespace nd4jhip
