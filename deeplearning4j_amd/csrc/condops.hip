// The legacy ops built on a "match condition" read from extraParams (libnd4j/include/ops/ops.h):
//   MatchConditionBool (TransformBool 5, :1800-1845)      z = cond(x)                       params [compare, eps, mode]
//   CompareAndSetTransform (TransformSame 13, :845-940)   z = cond(x) ? set : x             params [compare, set, eps, mode]
//   CompareAndSet (Pairwise 12 / Scalar 33, :719-840)     z = cond(y) ? y : x               params [compare, -, eps, mode]
//   CompareAndReplace (Pairwise 13, :593-715)             z = cond(x) ? y : x               params [compare, -, eps, mode]
//   MatchCondition (ReduceLong 2, :2430-2500)             count of cond(x) per sub-array    params [compare, eps, mode]
// and, through the same elementwise kernel, the three pairwise ops whose extraParams hold plain numbers:
//   Axpy (Pairwise 10, :328-333)                          z = p0 x + y (one fused multiply-add in the array's type)
//   BinaryRelativeError (Pairwise 25, :2218-2270)         z = re(x, y) > p0 ? 1 : 0,  re = |x - y| / (|x| + |y|), 0 for two zeros
//   BinaryMinimumAbsoluteRelativeError (26, :2274-2340)   z = re(x, y) > p0 && !(|x - y| < p1) ? 1 : 0
//   FirstIndex / LastIndex (IndexReduce 4 / 5, :2061-2150) first / last position with cond(x), -1 when none
// and the members of the bool tables (pairwise / scalar / broadcast, BOOL result) that are more than a comparison:
//   Epsilon (3, :1755-1790)                               |x - y| <= p0 when parameters are given, else <= 1e-5 (as the type holds it)
//   And / Or / Xor (7 / 8 / 9, :1051-1063, :1896-1925)    on "differs from p0" when parameters are given, else on "is not zero"
// The sixteen modes: 0 |v - c| <= eps, 1 |v - c| > eps, 2 <, 3 >, 4 <=, 5 >=, 6 |v| < c, 7 |v| > c, 8 isinf, 9 isnan, 10 ==, 11 !=,
// 12 |v| >= c, 13 |v| <= c, 14 finite, 15 inf or nan.  Comparisons run in the array's own type: the difference of mode 0 / 1
// is rounded through a 16-bit storage type as the reference's half / bfloat16 operators round it.
// The parameters arrive by value (the facade fetches them from extraParams).  Type-agnostic correctness kernels.
#include "anyio.h"
#include "device.h"
#include "kernels.h"
#include "runtime.h"

namespace nd4jhip {

__device__ __forceinline__ double sub_in_type(double a, double b, int dt) {
  if (dt == DOUBLE || dt == INT32 || dt == INT64 || dt == BOOL) return a - b;
  const float d = (float)a - (float)b;
  return (dt == HALF || dt == BFLOAT16) ? (double)round_as(d, dt) : (double)d;
}
// |a - b| / (|a| + |b|) in the array's type, 0 for two zeros (math/templatemath.h:1144-1153)
__device__ __forceinline__ double rel_err_in_type(double a, double b, int dt) {
  if (a == 0.0 && b == 0.0) return 0.0;
  if (dt == DOUBLE) return fabs(a - b) / (fabs(a) + fabs(b));
  const float fa = (float)a, fb = (float)b;
  return (double)round_as(fabsf(fa - fb) / (fabsf(fa) + fabsf(fb)), dt);
}
__device__ __forceinline__ bool cond_holds(const CondParams& c, double v) {
  const bool inf = (v - v) != (v - v) && v == v, nan = v != v;
  switch (c.mode) {
    case 0: return fabs(sub_in_type(v, c.compare, c.xdt)) <= c.eps;
    case 1: return fabs(sub_in_type(v, c.compare, c.xdt)) > c.eps;
    case 2: return v < c.compare;
    case 3: return v > c.compare;
    case 4: return v <= c.compare;
    case 5: return v >= c.compare;
    case 6: return fabs(v) < c.compare;
    case 7: return fabs(v) > c.compare;
    case 8: return inf;
    case 9: return nan;
    case 10: return v == c.compare;
    case 11: return v != c.compare;
    case 12: return fabs(v) >= c.compare;
    case 13: return fabs(v) <= c.compare;
    case 14: return !(inf || nan);
    case 15: return inf || nan;
    default: return false;
  }
}

__global__ __launch_bounds__(256) void cond_ew(int kind, CondParams c, DevShape sz, DevShape sx, DevShape sy, int zdt, int ydt, void* __restrict__ z,
                                               const void* __restrict__ x, const void* __restrict__ y, LongType n, double scalar, int hasScalar) {
  const LongType step = (LongType)gridDim.x * 256;
  for (LongType i = (LongType)blockIdx.x * 256 + threadIdx.x; i < n; i += step) {
    const double a = load_any(x, c.xdt, walk<LongType>(sx, i));
    double b = scalar, r;
    if (kind >= C_SET && !hasScalar) b = load_any(y, ydt, walk<LongType>(sy, i));
    switch (kind) {
      case C_MATCH_BOOL: r = cond_holds(c, a) ? 1.0 : 0.0; break;
      case C_SET_TRANSFORM: r = cond_holds(c, a) ? c.set : a; break;
      case C_SET: r = cond_holds(c, b) ? b : a; break;          // the second operand is the one tested
      case C_REPLACE: r = cond_holds(c, a) ? b : a; break;
      case C_AXPY: r = c.xdt == DOUBLE ? fma(c.compare, a, b) : (double)fmaf((float)c.compare, (float)a, (float)b); break;   // alpha x + y
      case C_BIN_REL_ERR: r = rel_err_in_type(a, b, c.xdt) > c.compare ? 1.0 : 0.0; break;
      case C_BIN_MIN_ABS_REL_ERR:                               // relative AND absolute threshold exceeded
        r = rel_err_in_type(a, b, c.xdt) > c.compare ? (fabs(sub_in_type(a, b, c.xdt)) < c.set ? 0.0 : 1.0) : 0.0;
        break;
      case C_BOOL_EPSILON: {                                    // |a - b| <= params[0] if given, else <= 1e-5 -- both held in the array's type
        const double ad = fabs(sub_in_type(a, b, c.xdt));
        r = ((c.mode && ad <= c.compare) || ad <= c.eps) ? 1.0 : 0.0;
        break;
      }
      case C_BOOL_AND: r = (c.mode ? (a != c.compare && b != c.compare) : (a != 0.0 && b != 0.0)) ? 1.0 : 0.0; break;
      case C_BOOL_OR: r = (c.mode ? (a != c.compare || b != c.compare) : (a != 0.0 || b != 0.0)) ? 1.0 : 0.0; break;
      default:                                                  // C_BOOL_XOR
        r = (c.mode ? ((a == c.compare) != (b == c.compare)) : ((a != 0.0) != (b != 0.0))) ? 1.0 : 0.0;
        break;
    }
    store_any(z, zdt, walk<LongType>(sz, i), r);
  }
}

void launchCondElementwise(hipStream_t s, CondKind kind, const CondParams& c, DataType ydt, DataType zdt, const void* x, const void* y, void* z,
                           const EwPlan& p, double scalar, bool hasScalar) {
  if (p.length == 0) return;
  LongType blocks = (p.length + 255) / 256;
  if (blocks > 4096) blocks = 4096;
  const bool binary = kind >= C_SET;
  hipLaunchKernelGGL(cond_ew, dim3((unsigned)blocks), dim3(256), 0, s, (int)kind, c, p.own[0], p.own[1], binary && !hasScalar ? p.own[2] : p.own[1], (int)zdt,
                     (int)ydt, z, x, binary && !hasScalar ? y : x, p.length, scalar, hasScalar ? 1 : 0);
  HIP_CHECK(hipGetLastError());
}

// ---- reductions: count of matches, first / last matching position --------------------------------------------------------
struct CondReduceArgs {
  DevShape outer, inner, zOuter;
  LongType outerLen, innerLen, segLen;
  int splits, kind, zdt, zLinear;
};
__device__ __forceinline__ LongType cr_merge(int kind, LongType a, LongType b) {
  if (kind == CR_COUNT) return a + b;
  if (a < 0) return b;
  if (b < 0) return a;
  return kind == CR_FIRST ? (a < b ? a : b) : (a > b ? a : b);
}
__global__ __launch_bounds__(256) void cond_reduce_partial(CondReduceArgs a, CondParams c, const void* __restrict__ x, void* __restrict__ z,
                                                           LongType* __restrict__ partials) {
  __shared__ LongType lv[256];
  const LongType unit = blockIdx.x, row = unit / a.splits;
  const int split = (int)(unit - row * a.splits), t = threadIdx.x;
  const LongType base = walk<LongType>(a.outer, row);
  const LongType j0 = (LongType)split * a.segLen;
  LongType j1 = j0 + a.segLen;
  if (j1 > a.innerLen) j1 = a.innerLen;
  const bool linear = a.inner.rank == 1;
  const LongType st = linear ? a.inner.stride[0] : 0;
  LongType acc = a.kind == CR_COUNT ? 0 : -1;
  for (LongType q = j0 + t; q < j1; q += 256) {
    const bool hit = cond_holds(c, load_any(x, c.xdt, base + (linear ? q * st : walk<LongType>(a.inner, q))));
    if (hit) acc = a.kind == CR_COUNT ? acc + 1 : cr_merge(a.kind, acc, q);
  }
  lv[t] = acc;
  __syncthreads();
  for (int w = 128; w > 0; w >>= 1) {
    if (t < w) lv[t] = cr_merge(a.kind, lv[t], lv[t + w]);
    __syncthreads();
  }
  if (t != 0) return;
  if (a.splits == 1) store_any(z, a.zdt, a.zLinear ? row : walk<LongType>(a.zOuter, row), (double)lv[0]);
  else partials[unit] = lv[0];
}
__global__ __launch_bounds__(256) void cond_reduce_finish(CondReduceArgs a, const LongType* __restrict__ partials, void* __restrict__ z) {
  const LongType row = (LongType)blockIdx.x * 256 + threadIdx.x;
  if (row >= a.outerLen) return;
  LongType acc = a.kind == CR_COUNT ? 0 : -1;
  for (int s = 0; s < a.splits; s++) acc = cr_merge(a.kind, acc, partials[row * a.splits + s]);
  store_any(z, a.zdt, a.zLinear ? row : walk<LongType>(a.zOuter, row), (double)acc);
}

void launchCondReduce(hipStream_t st, CondReduceKind kind, const CondParams& c, DataType zdt, const void* x, void* z, const ReducePlan& p, void* scratch,
                      size_t scratchBytes) {
  if (p.outerLen == 0) return;
  ND4J_REQUIRE(zdt == INT64 || zdt == INT32, "match-condition reduction: output must be INT32 or INT64");
  CondReduceArgs a;
  a.outer = p.outer; a.inner = p.inner; a.zOuter = p.zOuter;
  a.outerLen = p.outerLen; a.innerLen = p.innerLen;
  a.kind = (int)kind; a.zdt = (int)zdt; a.zLinear = p.zLinear ? 1 : 0;
  LongType splits = 1;
  if (p.outerLen < 1024 && p.innerLen > 16384) {
    splits = std::min<LongType>((2048 + p.outerLen - 1) / p.outerLen, (p.innerLen + 8191) / 8192);
    const LongType cap = (LongType)(scratchBytes / sizeof(LongType)) / p.outerLen;
    splits = std::max<LongType>(1, std::min(splits, cap));
  }
  a.splits = (int)splits;
  a.segLen = (p.innerLen + splits - 1) / splits;
  ND4J_REQUIRE(p.outerLen * splits < (1LL << 31), "reduce: too many outputs");
  hipLaunchKernelGGL(cond_reduce_partial, dim3((unsigned)(p.outerLen * splits)), dim3(256), 0, st, a, c, x, z, (LongType*)scratch);
  if (splits > 1) hipLaunchKernelGGL(cond_reduce_finish, dim3((unsigned)((p.outerLen + 255) / 256)), dim3(256), 0, st, a, (const LongType*)scratch, z);
  HIP_CHECK(hipGetLastError());
}

}  // namespace nd4jhip
