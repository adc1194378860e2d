// Integer and boolean arrays on the legacy loops: pairwise / scalar / broadcast arithmetic, same-type transforms,
// ReduceSame and IndexReduce.  The reference instantiates those loops for every common type
// (libnd4j/include/legacy/cpu/NativeOpExecutioner_pairwise_floats.cpp:23-68, loops/cpu/reduce/reduce_same.hpp:156-193,
// loops/cpu/indexreduce.hpp:98-140); a decoder graph adds INT64 position ids and takes the arg-max of integer arrays.
//
// All arithmetic runs in 64-bit integers and is narrowed on the store.  For +, -, * and the comparisons that is the
// same result as arithmetic in the narrower type (two's complement wrap-around); divisions take the operands as the
// storage type holds them.  A zero divisor gives 0 (the reference's CPU loop traps there).
// HBM-bound, not tuned beyond a 16-byte vector path for dense INT32 / INT64 operands.
#include "device.h"
#include "kernels.h"
#include "runtime.h"

namespace nd4jhip {

bool isIntLike(DataType t) {
  switch (t) {
    case BOOL: case INT8: case UINT8: case INT16: case UINT16: case INT32: case UINT32: case INT64: case UINT64: return true;
    default: return false;
  }
}

__device__ __forceinline__ LongType load_i64(const void* p, int dt, LongType off) {
  switch (dt) {
    case BOOL: case UINT8: return ((const unsigned char*)p)[off];
    case INT8: return ((const signed char*)p)[off];
    case INT16: return ((const short*)p)[off];
    case UINT16: return ((const unsigned short*)p)[off];
    case INT32: return ((const int*)p)[off];
    case UINT32: return ((const unsigned*)p)[off];
    default: return ((const LongType*)p)[off];   // INT64, UINT64
  }
}
__device__ __forceinline__ void store_i64(void* p, int dt, LongType off, LongType v) {
  switch (dt) {
    case BOOL: ((unsigned char*)p)[off] = v != 0; break;
    case UINT8: case INT8: ((unsigned char*)p)[off] = (unsigned char)v; break;
    case INT16: case UINT16: ((unsigned short*)p)[off] = (unsigned short)v; break;
    case INT32: case UINT32: ((unsigned*)p)[off] = (unsigned)v; break;
    default: ((LongType*)p)[off] = v; break;
  }
}

__device__ __forceinline__ LongType iabs(LongType a) { return a < 0 ? -a : a; }
__device__ __forceinline__ LongType ifloordiv(LongType a, LongType b) {
  if (b == 0) return 0;
  LongType q = a / b;
  if ((a % b != 0) && ((a < 0) != (b < 0))) q--;
  return q;
}
// a = element of x, b = element of y or the scalar.  Formulas: ops/ops.h of the reference with integer X, Y, Z.
__device__ __forceinline__ LongType int_binary(int k, LongType a, LongType b) {
  switch (k) {
    case P_ADD: return a + b;                                   // ops.h:56
    case P_SUB: return a - b;                                   // ops.h:57
    case P_MUL: return a * b;                                   // ops.h:58
    case P_DIV: case P_SAFE_DIVIDE: case P_DIVIDE_NO_NAN: case P_TRUNCATE_DIV: return b == 0 ? 0 : a / b;   // ops.h:59,232-245
    case P_RSUB: return b - a;                                  // ops.h:63
    case P_RDIV: return a == 0 ? 0 : b / a;                     // ops.h:64
    case P_COPY: return b;                                      // ops.h:312-317
    case P_MAX: return a > b ? a : b;                           // ops.h:103-108
    case P_MIN: return a < b ? a : b;                           // ops.h:110-115
    case P_SQSUB: return (a - b) * (a - b);                     // ops.h:174
    case P_SQ_RSUB: return (b - a) * (b - a);
    case P_AMAX: return iabs(a) > iabs(b) ? a : b;              // ops.h:89-94
    case P_AMIN: return iabs(a) < iabs(b) ? a : b;              // ops.h:96-101
    case P_FLOOR_DIV: return ifloordiv(a, b);                   // op_macros_special.h:87-93
    case P_FLOOR_MOD: {                                         // ops.h:260-267: fmod, shifted by b when the signs differ
      if (b == 0) return 0;
      const LongType m = a % b;
      return ((a < 0) == (b < 0)) ? m : (m + b) % b;
    }
    case P_MOD: case P_TRUNCATE_MOD: case P_FMOD: return b == 0 ? 0 : a % b;   // ops.h:247-252,1708-1715: d1 - (d1 / d2) * d2 in integers
    case P_REVERSE_MOD: return a == 0 ? 0 : b % a;              // ops.h:1747-1752
    case P_LOGICAL_OR: return a | b;                            // ops.h:2423-2428
    case P_LOGICAL_XOR: return (a | b) & ~(a & b);              // ops.h:2407-2412
    case P_LOGICAL_NOT: return !(a && b);                       // ops.h:2399-2404
    case P_LOGICAL_AND: return a & b;                           // ops.h:2415-2420
    case P_RELU: return a < b ? b : a;                          // ops.h:1108-1112
    case P_STEP: case P_RELU_D: return a > b ? 1 : 0;           // ops.h:347-350
    case P_EQ: return a == b;                                   // ops.h:181-186
    case P_NE: return a != b;
    case P_GT: return a > b;
    case P_GE: return a >= b;
    case P_LT: return a < b;
    case P_LE: return a <= b;
    default: return a;
  }
}
bool intBinarySupported(PairwiseKind k) {
  switch (k) {
    case P_ADD: case P_SUB: case P_MUL: case P_DIV: case P_SAFE_DIVIDE: case P_DIVIDE_NO_NAN: case P_TRUNCATE_DIV: case P_RSUB: case P_RDIV:
    case P_COPY: case P_MAX: case P_MIN: case P_SQSUB: case P_SQ_RSUB: case P_AMAX: case P_AMIN: case P_FLOOR_DIV: case P_FLOOR_MOD: case P_MOD:
    case P_TRUNCATE_MOD: case P_FMOD: case P_REVERSE_MOD: case P_LOGICAL_OR: case P_LOGICAL_XOR: case P_LOGICAL_NOT: case P_LOGICAL_AND:
    case P_RELU: case P_STEP: case P_RELU_D: case P_EQ: case P_NE: case P_GT: case P_GE: case P_LT: case P_LE: return true;
    default: return false;
  }
}
__device__ __forceinline__ LongType int_unary(int k, LongType x) {
  switch (k) {
    case U_ABS: return iabs(x);                                 // ops.h:192
    case U_NEG: return -x;                                      // ops.h:202
    case U_SQUARE: return x * x;                                // ops.h:203
    case U_CUBE: return x * x * x;                              // ops.h:204
    case U_ONE_MINUS: return 1 - x;                             // ops.h:206
    case U_RECIPROCAL: return x == 0 ? 0 : 1 / x;               // ops.h:207
    case U_ONES: return 1;                                      // ops.h:481
    case U_TIMES_ONE_MINUS: return x * (1 - x);                 // ops.h:1165
    case U_SIGN_REF: return x != 0 ? 1 : -1;                    // ops.h:217-219: the macro tests the sign expression
    case U_IS_POSITIVE: return x > 0;                           // TransformBool, ops.h:1140-1163
    case U_IS_NEGATIVE: return x < 0;
    case U_NOT: return x == 0;
    case U_IS_FINITE: return 1;
    case U_IS_INF: case U_IS_NAN: case U_IS_INF_OR_NAN: return 0;
    default: return x;                                          // Identity / Copy / Round / Ceil / Floor / Rint
  }
}
bool intUnarySupported(UnaryKind k) {
  switch (k) {
    case U_ABS: case U_NEG: case U_SQUARE: case U_CUBE: case U_ONE_MINUS: case U_RECIPROCAL: case U_ONES: case U_TIMES_ONE_MINUS:
    case U_IDENTITY: case U_ROUND: case U_CEIL: case U_FLOOR: case U_RINT: case U_SIGN_REF:
    case U_IS_POSITIVE: case U_IS_NEGATIVE: case U_NOT: case U_IS_FINITE: case U_IS_INF: case U_IS_NAN: case U_IS_INF_OR_NAN: return true;
    default: return false;
  }
}

// UINT64 travels through the signed 64-bit arithmetic above bit for bit, which is the right result only where wrap-around
// arithmetic does not look at the sign: values of 2^63 and more would compare, divide and take remainders as negative
// numbers.  Those ops are refused for UINT64 operands rather than computed wrongly.
static bool signAgnosticBinary(PairwiseKind k) {
  switch (k) {
    case P_ADD: case P_SUB: case P_MUL: case P_RSUB: case P_COPY: case P_SQSUB: case P_SQ_RSUB: case P_LOGICAL_OR: case P_LOGICAL_XOR:
    case P_LOGICAL_NOT: case P_LOGICAL_AND: case P_EQ: case P_NE: return true;
    default: return false;
  }
}
static bool signAgnosticUnary(UnaryKind k) {
  switch (k) {
    case U_NEG: case U_SQUARE: case U_CUBE: case U_ONE_MINUS: case U_ONES: case U_TIMES_ONE_MINUS: case U_IDENTITY: case U_ROUND: case U_CEIL:
    case U_FLOOR: case U_RINT: case U_SIGN_REF: case U_NOT: case U_IS_FINITE: case U_IS_INF: case U_IS_NAN: case U_IS_INF_OR_NAN: return true;
    default: return false;
  }
}

// ---- elementwise --------------------------------------------------------------------------------------------------------
// any strides, any integer types per operand; NIN = 1: unary op k (UnaryKind), NIN = 2: binary op k (PairwiseKind) with
// y or, when hasScalar, the scalar
template <int NIN>
__global__ __launch_bounds__(256) void int_ew(int k, DevShape sz, DevShape sx, DevShape sy, int zdt, int xdt, int ydt, void* __restrict__ z,
                                              const void* __restrict__ x, const void* __restrict__ y, LongType n, LongType scalar, int hasScalar) {
  const LongType step = (LongType)gridDim.x * 256;
  for (LongType i = (LongType)blockIdx.x * 256 + threadIdx.x; i < n; i += step) {
    const LongType a = load_i64(x, xdt, walk<LongType>(sx, i));
    LongType r;
    if (NIN == 1) r = int_unary(k, a);
    else r = int_binary(k, a, hasScalar ? scalar : load_i64(y, ydt, walk<LongType>(sy, i)));
    store_i64(z, zdt, walk<LongType>(sz, i), r);
  }
}
// dense operands of one type (INT32 or INT64): one 16-byte vector per thread
template <typename T, int NIN>
__global__ __launch_bounds__(256) void int_ew_contig(int k, const T* __restrict__ x, const T* __restrict__ y, T* __restrict__ z, LongType n,
                                                     LongType scalar, int hasScalar) {
  constexpr int V = 16 / sizeof(T);
  using VT = Vec<T, V>;
  const LongType nvec = n / V, i = (LongType)blockIdx.x * 256 + threadIdx.x;
  if (i < nvec) {
    VT a = reinterpret_cast<const VT*>(x)[i], b = a, out;
    if (NIN > 1 && !hasScalar) b = reinterpret_cast<const VT*>(y)[i];
#pragma unroll
    for (int e = 0; e < V; e++)
      out.v[e] = (T)(NIN == 1 ? int_unary(k, (LongType)a.v[e]) : int_binary(k, (LongType)a.v[e], hasScalar ? scalar : (LongType)b.v[e]));
    reinterpret_cast<VT*>(z)[i] = out;
  }
  const LongType tail = nvec * V + i;
  if (tail < n) z[tail] = (T)(NIN == 1 ? int_unary(k, (LongType)x[tail]) : int_binary(k, (LongType)x[tail], hasScalar ? scalar : (LongType)y[tail]));
}

static unsigned gridCap(LongType work) {
  LongType blocks = (work + 255) / 256;
  if (blocks > 256 * 16) blocks = 256 * 16;
  return (unsigned)(blocks < 1 ? 1 : blocks);
}
static bool al16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

// k: UnaryKind when y == nullptr and !hasScalar, else PairwiseKind
void launchIntElementwise(hipStream_t s, int k, bool binary, DataType xdt, DataType ydt, DataType zdt, const void* x, const void* y, void* z,
                          const EwPlan& p, LongType scalar, bool hasScalar) {
  if (p.length == 0) return;
  ND4J_REQUIRE(isIntLike(xdt) && isIntLike(zdt) && (!binary || hasScalar || isIntLike(ydt)), "integer elementwise op: integer or bool operands only");
  if (binary) ND4J_REQUIRE(intBinarySupported((PairwiseKind)k), "this pairwise / scalar / broadcast op is not implemented for integer arrays in nd4j-hip");
  else ND4J_REQUIRE(intUnarySupported((UnaryKind)k), "this transform is not implemented for integer arrays in nd4j-hip");
  if (xdt == UINT64 || zdt == UINT64 || (binary && !hasScalar && ydt == UINT64)) {
    ND4J_REQUIRE(!hasScalar, "scalar ops on UINT64 arrays are not implemented in nd4j-hip (the scalar travels as a signed 64-bit value)");
    ND4J_REQUIRE(binary ? signAgnosticBinary((PairwiseKind)k) : signAgnosticUnary((UnaryKind)k),
                 "this op orders, divides or takes remainders of its operands, which nd4j-hip computes in signed 64-bit arithmetic: not implemented for UINT64 arrays");
  }
  const bool same = xdt == zdt && (!binary || hasScalar || ydt == zdt);
  if (same && p.sameShape && p.contiguous && (zdt == INT32 || zdt == INT64) && al16(x) && al16(z) && (!binary || hasScalar || al16(y))) {
    const LongType V = zdt == INT32 ? 4 : 2;
    const unsigned grid = (unsigned)((p.length / V + 256) / 256);
    const void* yy = binary && !hasScalar ? y : x;
#define INT_CONTIG(T, NIN) hipLaunchKernelGGL((int_ew_contig<T, NIN>), dim3(grid), dim3(256), 0, s, k, (const T*)x, (const T*)yy, (T*)z, p.length, scalar, hasScalar ? 1 : 0)
    if (zdt == INT32) { if (binary) INT_CONTIG(int, 2); else INT_CONTIG(int, 1); }
    else { if (binary) INT_CONTIG(LongType, 2); else INT_CONTIG(LongType, 1); }
#undef INT_CONTIG
  } else if (binary) {
    hipLaunchKernelGGL((int_ew<2>), dim3(gridCap(p.length)), dim3(256), 0, s, k, p.own[0], p.own[1], hasScalar ? p.own[1] : p.own[2], (int)zdt, (int)xdt,
                       (int)ydt, z, x, hasScalar ? x : y, p.length, scalar, hasScalar ? 1 : 0);
  } else {
    hipLaunchKernelGGL((int_ew<1>), dim3(gridCap(p.length)), dim3(256), 0, s, k, p.own[0], p.own[1], p.own[1], (int)zdt, (int)xdt, (int)xdt, z, x, x,
                       p.length, (LongType)0, 0);
  }
  HIP_CHECK(hipGetLastError());
}

// ---- reductions ------------------------------------------------------------------------------------------------------------
// One block per (output, split of the reduced run).  Value kinds keep one 64-bit accumulator; index kinds keep
// (value, position) with the reference's rule: strictly better replaces, so the first extreme wins
// (ops/op_macros_index_reduce.h:18-72).  Partials of split runs go to the scratch area as (value, position) pairs and
// are merged in split order.
struct IntReduceArgs {
  DevShape outer, inner, zOuter;
  LongType outerLen, innerLen, segLen;
  int splits, kind, isIndex, xdt, zdt, zLinear;
};
enum IntReduceKind : int { IR_SUM, IR_MAX, IR_MIN, IR_PROD, IR_ASUM, IR_AMAX, IR_AMIN };

__device__ __forceinline__ LongType ir_identity(int kind, int isIndex) {
  if (isIndex) return 0;
  switch (kind) {
    case IR_MAX: return (LongType)0x8000000000000000ULL;
    case IR_MIN: return 0x7fffffffffffffffLL;
    case IR_AMIN: return 0x7fffffffffffffffLL;
    case IR_PROD: return 1;
    default: return 0;   // Sum, ASum, AMax
  }
}
__device__ __forceinline__ LongType ir_pre(int kind, int isIndex, LongType v) {
  if (isIndex) return (kind == I_AMAX || kind == I_AMIN) ? iabs(v) : v;
  return (kind == IR_ASUM || kind == IR_AMAX || kind == IR_AMIN) ? iabs(v) : v;
}
__device__ __forceinline__ LongType ir_merge(int kind, LongType a, LongType b) {
  switch (kind) {
    case IR_MAX: case IR_AMAX: return a > b ? a : b;
    case IR_MIN: case IR_AMIN: return a < b ? a : b;
    case IR_PROD: return a * b;
    default: return a + b;
  }
}
// does candidate (v, i) beat (bv, bi): better value, or the same value at an earlier position
__device__ __forceinline__ bool ir_better(int kind, LongType v, LongType i, LongType bv, LongType bi) {
  if (bi < 0) return true;
  const bool wantMax = kind == I_MAX || kind == I_AMAX;
  if (v != bv) return wantMax ? v > bv : v < bv;
  return i < bi;
}
__global__ __launch_bounds__(256) void int_reduce_partial(IntReduceArgs a, const void* __restrict__ x, void* __restrict__ z, LongType* __restrict__ partials) {
  __shared__ LongType lv[256];
  __shared__ LongType li[256];
  const LongType unit = blockIdx.x, row = unit / a.splits;
  const int split = (int)(unit - row * a.splits), t = threadIdx.x;
  const LongType base = walk<LongType>(a.outer, row);
  const LongType j0 = (LongType)split * a.segLen;
  LongType j1 = j0 + a.segLen;
  if (j1 > a.innerLen) j1 = a.innerLen;
  const bool linear = a.inner.rank == 1;
  const LongType st = linear ? a.inner.stride[0] : 0;
  LongType acc = ir_identity(a.kind, a.isIndex), pos = -1;
  for (LongType q = j0 + t; q < j1; q += 256) {
    const LongType v = ir_pre(a.kind, a.isIndex, load_i64(x, a.xdt, base + (linear ? q * st : walk<LongType>(a.inner, q))));
    if (a.isIndex) { if (ir_better(a.kind, v, q, acc, pos)) { acc = v; pos = q; } }
    else acc = ir_merge(a.kind, acc, v);
  }
  lv[t] = acc; li[t] = pos;
  __syncthreads();
  for (int w = 128; w > 0; w >>= 1) {
    if (t < w) {
      if (a.isIndex) { if (li[t + w] >= 0 && ir_better(a.kind, lv[t + w], li[t + w], lv[t], li[t])) { lv[t] = lv[t + w]; li[t] = li[t + w]; } }
      else lv[t] = ir_merge(a.kind, lv[t], lv[t + w]);
    }
    __syncthreads();
  }
  if (t != 0) return;
  if (a.splits == 1) {
    const LongType zo = a.zLinear ? row : walk<LongType>(a.zOuter, row);
    store_i64(z, a.zdt, zo, a.isIndex ? (li[0] < 0 ? 0 : li[0]) : lv[0]);
  } else {
    partials[unit * 2] = lv[0]; partials[unit * 2 + 1] = li[0];
  }
}
__global__ __launch_bounds__(256) void int_reduce_finish(IntReduceArgs a, const LongType* __restrict__ partials, void* __restrict__ z) {
  const LongType row = (LongType)blockIdx.x * 256 + threadIdx.x;
  if (row >= a.outerLen) return;
  LongType acc = ir_identity(a.kind, a.isIndex), pos = -1;
  for (int s = 0; s < a.splits; s++) {
    const LongType v = partials[(row * a.splits + s) * 2], i = partials[(row * a.splits + s) * 2 + 1];
    if (a.isIndex) { if (i >= 0 && ir_better(a.kind, v, i, acc, pos)) { acc = v; pos = i; } }
    else acc = ir_merge(a.kind, acc, v);
  }
  const LongType zo = a.zLinear ? row : walk<LongType>(a.zOuter, row);
  store_i64(z, a.zdt, zo, a.isIndex ? (pos < 0 ? 0 : pos) : acc);
}

// kind: ReduceKind (R_SUM .. R_AMIN) for value reductions, IndexKind for index reductions
void launchIntReduce(hipStream_t st, int kind, bool isIndex, DataType xdt, DataType zdt, const void* x, void* z, const ReducePlan& p, void* scratch,
                     size_t scratchBytes) {
  if (p.outerLen == 0) return;
  ND4J_REQUIRE(isIntLike(xdt) && isIntLike(zdt), "integer reduction: integer or bool arrays only");
  // signed 64-bit accumulators: sums and products wrap around as UINT64's do, extremes and their positions would not be UINT64's
  ND4J_REQUIRE(xdt != UINT64 || (!isIndex && ((ReduceKind)kind == R_SUM || (ReduceKind)kind == R_PROD)),
               "extremes, absolute values and index reductions of UINT64 arrays are not implemented in nd4j-hip (signed 64-bit arithmetic)");
  IntReduceArgs a;
  a.outer = p.outer; a.inner = p.inner; a.zOuter = p.zOuter;
  a.outerLen = p.outerLen; a.innerLen = p.innerLen;
  a.isIndex = isIndex ? 1 : 0; a.xdt = (int)xdt; a.zdt = (int)zdt; a.zLinear = p.zLinear ? 1 : 0;
  if (isIndex) a.kind = kind;
  else switch ((ReduceKind)kind) {
    case R_SUM: a.kind = IR_SUM; break; case R_MAX: a.kind = IR_MAX; break; case R_MIN: a.kind = IR_MIN; break; case R_PROD: a.kind = IR_PROD; break;
    case R_ASUM: a.kind = IR_ASUM; break; case R_AMAX: a.kind = IR_AMAX; break; case R_AMIN: a.kind = IR_AMIN; break;
    default: ND4J_THROW("this reduction is not implemented for integer arrays in nd4j-hip");
  }
  LongType splits = 1;
  if (p.outerLen < 1024 && p.innerLen > 16384) {
    splits = std::min<LongType>((2048 + p.outerLen - 1) / p.outerLen, (p.innerLen + 8191) / 8192);
    const LongType cap = (LongType)(scratchBytes / (2 * sizeof(LongType))) / p.outerLen;
    splits = std::max<LongType>(1, std::min(splits, cap));
  }
  a.splits = (int)splits;
  a.segLen = (p.innerLen + splits - 1) / splits;
  ND4J_REQUIRE(p.outerLen * splits < (1LL << 31), "reduce: too many outputs");
  hipLaunchKernelGGL(int_reduce_partial, dim3((unsigned)(p.outerLen * splits)), dim3(256), 0, st, a, x, z, (LongType*)scratch);
  if (splits > 1) hipLaunchKernelGGL(int_reduce_finish, dim3((unsigned)((p.outerLen + 255) / 256)), dim3(256), 0, st, a, (const LongType*)scratch, z);
  HIP_CHECK(hipGetLastError());
}

}  // namespace nd4jhip
