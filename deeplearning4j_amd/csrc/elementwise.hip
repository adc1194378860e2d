// Elementwise kernels: unary transforms and pairwise transforms.
//
// Three variants, picked by the host plan:
//   contig  - all operands dense and unit-stride: 16-byte loads/stores, four vectors in flight per
//             operand and thread, grid sized to a few blocks per CU.  HBM-bound; algorithmic bytes
//             = (inputs + 1) * sizeof(T) per element.
//   nd      - operands share one (collapsed) shape but have their own strides: the coordinate
//             decomposition is done once per thread and shared by all operands; when the innermost
//             stride is 1 everywhere the thread moves a 16-byte vector.
//   generic - operands of different shapes and/or dtypes (equal length): every operand walks its
//             own shape, loads convert at run time.  Correctness path.
//
// Functor formulas follow the reference's simdOps (libnd4j/include/ops/ops.h) and sd::math
// (libnd4j/include/math/templatemath.h); the citations sit on each functor.
#include "device.h"
#include "kernels.h"
#include "runtime.h"

namespace nd4jhip {

// ---- functors --------------------------------------------------------------------------------------
template <typename A> __device__ __forceinline__ A d_exp(A x);
template <> __device__ __forceinline__ float d_exp<float>(float x) { return expf(x); }
template <> __device__ __forceinline__ double d_exp<double>(double x) { return exp(x); }

// sd_sigmoid = 1 / (1 + exp(-x))                                   templatemath.h:225-229
// (float: the exponential and the reciprocal come from fast_exp / fast_rcp, a few ulp in total, so that the
// bf16/fp16 flavours stay memory-bound rather than instruction-bound)
template <typename A> __device__ __forceinline__ A d_sigmoid(A x) { return fast_rcp((A)1 + fast_exp(-x)); }
// sd_tanh<float> = copysign(1,x) * (1-p)/(1+p), p = e^(-2|x|)       templatemath.h:1206-1223
__device__ __forceinline__ float d_tanh(float x) {
  float ax = fabsf(x);
  float p = fast_exp(-2.f * ax);
  return copysignf((1.f - p) * fast_rcp(1.f + p), x);
}
// generic sd_tanh: (p-1)/(p+1), p = e^(2x) for x <= 0, mirrored otherwise   templatemath.h:1183-1204
__device__ __forceinline__ double d_tanh(double x) {
  if (x <= 0) { double p = exp(2.0 * x); return (p - 1.0) / (p + 1.0); }
  double p = exp(-2.0 * x);
  return (1.0 - p) / (1.0 + p);
}

template <int K> struct Unary;
#define UNARY(K, EXPR) \
  template <> struct Unary<K> { template <typename A> static __device__ __forceinline__ A apply(A x) { return EXPR; } }
__device__ __forceinline__ float d_cos(float x) { return cosf(x); }
__device__ __forceinline__ double d_cos(double x) { return cos(x); }
__device__ __forceinline__ float d_sin(float x) { return sinf(x); }
__device__ __forceinline__ double d_sin(double x) { return sin(x); }
__device__ __forceinline__ float d_log(float x) { return logf(x); }
__device__ __forceinline__ double d_log(double x) { return log(x); }
__device__ __forceinline__ float d_erf(float x) { return erff(x); }
__device__ __forceinline__ double d_erf(double x) { return erf(x); }
__device__ __forceinline__ float d_sqrt(float x) { return sqrtf(x); }
__device__ __forceinline__ double d_sqrt(double x) { return sqrt(x); }
__device__ __forceinline__ float d_abs(float x) { return fabsf(x); }
__device__ __forceinline__ double d_abs(double x) { return fabs(x); }
// PreciseGELU: x/2 * (1 + tanh(sqrt(2/pi) * (x + (0.044715 x)^3)))  -- the cube wraps 0.044715*x   ops.h:1015-1019
__device__ __forceinline__ float d_pgelu(float x) {
  const float sp = 0.79788458347320556640625f;  // sqrtf(2.0f / (float)M_PI)
  float c = 0.044715f * x;
  float xp = x + c * c * c;
  return (x / 2.f) * (1.f + d_tanh(sp * xp));
}
__device__ __forceinline__ double d_pgelu(double x) {
  const double sp = 0.7978845608028654;
  double c = 0.044715 * x;
  double xp = x + c * c * c;
  return (x / 2.0) * (1.0 + d_tanh(sp * xp));
}
UNARY(U_COS, d_cos(x));                                        // ops.h:194
UNARY(U_EXP, d_exp<A>(x));                                     // ops.h:195
UNARY(U_LOG, d_log(x));                                        // ops.h:197
UNARY(U_SIGMOID, d_sigmoid<A>(x));                             // ops.h:200
UNARY(U_SIN, d_sin(x));                                        // ops.h:198
UNARY(U_SOFTPLUS, d_log((A)1 + fast_exp(x)));                  // templatemath.h:272-274
UNARY(U_TANH, d_tanh(x));                                      // ops.h:199
UNARY(U_SWISH, x * d_sigmoid<A>(x));                           // ops.h:988-990
UNARY(U_ERF, d_erf(x));                                        // ops.h:361
UNARY(U_GELU, x * d_sigmoid<A>((A)1.702f * x));                // ops.h:1010-1012
UNARY(U_PRECISE_GELU, d_pgelu(x));
UNARY(U_SQRT, d_sqrt(x));                                      // ops.h:2200
UNARY(U_RSQRT, (A)1 / d_sqrt(x));                              // ops.h:2203-2205
UNARY(U_ABS, d_abs(x));                                        // ops.h:192
UNARY(U_NEG, -x);                                              // ops.h:202
UNARY(U_SQUARE, x * x);                                        // ops.h:203
UNARY(U_RECIPROCAL, (A)1 / x);                                 // ops.h:207
UNARY(U_IDENTITY, x);                                          // ops.h:205
UNARY(U_ONE_MINUS, (A)1 - x);                                  // ops.h:206
UNARY(U_CUBE, x * x * x);                                      // ops.h:204

template <int K> struct Pairwise;
#define PAIRWISE(K, EXPR) \
  template <> struct Pairwise<K> { template <typename A> static __device__ __forceinline__ A apply(A a, A b) { return EXPR; } }
PAIRWISE(P_ADD, a + b);              // ops.h:56
PAIRWISE(P_COPY, b);                 // CopyPws ops.h:312-317
PAIRWISE(P_DIV, a / b);              // ops.h:59
PAIRWISE(P_MUL, a * b);              // ops.h:58
PAIRWISE(P_RSUB, b - a);             // ops.h:63
PAIRWISE(P_SUB, a - b);              // ops.h:57
PAIRWISE(P_MAX, a > b ? a : b);      // ops.h:103-108
PAIRWISE(P_MIN, a < b ? a : b);      // ops.h:110-115
PAIRWISE(P_RDIV, b / a);             // ops.h:64
PAIRWISE(P_SQSUB, (a - b) * (a - b)); // ops.h:174

// ---- contiguous kernels ------------------------------------------------------------------------------
// One 16-byte vector per operand and thread, grid = one thread per vector: measured on MI355X this beats
// grid-stride loops with several vectors in flight.  NT = non-temporal loads/stores, chosen by the host when
// the operands together exceed what the 256 MB last-level cache can hold, so that streaming data does not
// evict itself (add over three 128 MiB arrays: 4.8 TB/s cached vs 6.8 TB/s non-temporal).
constexpr int EW_BLOCK = 256;

template <bool NT, typename VT>
__device__ __forceinline__ VT ld_stream(const VT* p) { return NT ? __builtin_nontemporal_load(p) : *p; }
template <bool NT, typename VT>
__device__ __forceinline__ void st_stream(VT* p, const VT& v) {
  if (NT) __builtin_nontemporal_store(v, p);
  else *p = v;
}

template <typename F, typename T, bool NT>
__global__ __launch_bounds__(EW_BLOCK) void unary_contig(const T* __restrict__ x, T* __restrict__ z, LongType n) {
  constexpr int V = 16 / sizeof(T);
  using IO = RawIO<T>;
  using RT = typename IO::raw;
  using A = typename Conv<T>::acc;
  const LongType nvec = n / V;
  const LongType i = (LongType)blockIdx.x * EW_BLOCK + threadIdx.x;
  if (i < nvec) {
    RT r = ld_stream<NT>(reinterpret_cast<const RT*>(x) + i);
    A vals[V];
    IO::unpack(r, vals);
#pragma unroll
    for (int e = 0; e < V; e++) vals[e] = F::template apply<A>(vals[e]);
    st_stream<NT>(reinterpret_cast<RT*>(z) + i, IO::pack(vals));
  }
  // scalar tail (fewer than V elements)
  const LongType tail = nvec * V + i;
  if (tail < n) z[tail] = Conv<T>::from(F::template apply<A>((A)to_float(x[tail])));
}

template <typename F, typename T, bool NT>
__global__ __launch_bounds__(EW_BLOCK) void pairwise_contig(const T* __restrict__ x, const T* __restrict__ y,
                                                            T* __restrict__ z, LongType n) {
  constexpr int V = 16 / sizeof(T);
  using IO = RawIO<T>;
  using RT = typename IO::raw;
  using A = typename Conv<T>::acc;
  const LongType nvec = n / V;
  const LongType i = (LongType)blockIdx.x * EW_BLOCK + threadIdx.x;
  if (i < nvec) {
    RT ra = ld_stream<NT>(reinterpret_cast<const RT*>(x) + i);
    RT rb = ld_stream<NT>(reinterpret_cast<const RT*>(y) + i);
    A a[V], b[V];
    IO::unpack(ra, a);
    IO::unpack(rb, b);
#pragma unroll
    for (int e = 0; e < V; e++) a[e] = F::template apply<A>(a[e], b[e]);
    st_stream<NT>(reinterpret_cast<RT*>(z) + i, IO::pack(a));
  }
  const LongType tail = nvec * V + i;
  if (tail < n) z[tail] = Conv<T>::from(F::template apply<A>((A)to_float(x[tail]), (A)to_float(y[tail])));
}
// ---- same-shape strided kernels ------------------------------------------------------------------------
struct NdArgs {
  int rank;                        // >= 1; dim rank-1 is the inner run
  LongType shape[MAX_DEV_RANK];
  LongType stride[3][MAX_DEV_RANK];
};

// One thread per chunk of VEC consecutive inner elements.  VEC > 1 requires unit inner strides, an inner
// extent divisible by VEC and VEC-aligned bases/outer strides (checked on the host).
template <typename F, typename T, int NIN, int VEC, typename I>
__global__ __launch_bounds__(EW_BLOCK) void ew_nd(NdArgs a, const T* __restrict__ x, const T* __restrict__ y,
                                                  T* __restrict__ z, I chunksPerRow, I totalChunks) {
  using A = typename Conv<T>::acc;
  using VT = Vec<T, VEC>;
  const I step = (I)gridDim.x * EW_BLOCK;
  for (I c = (I)blockIdx.x * EW_BLOCK + threadIdx.x; c < totalChunks; c += step) {
    I outer = c / chunksPerRow;
    I inner = (c - outer * chunksPerRow) * VEC;
    LongType oz = (LongType)inner * a.stride[0][a.rank - 1];
    LongType ox = (LongType)inner * a.stride[1][a.rank - 1];
    LongType oy = NIN > 1 ? (LongType)inner * a.stride[2][a.rank - 1] : 0;
#pragma unroll 1
    for (int d = a.rank - 2; d >= 0; d--) {
      I dim = (I)a.shape[d];
      I q = outer / dim;
      LongType cd = (LongType)(outer - q * dim);
      oz += cd * a.stride[0][d];
      ox += cd * a.stride[1][d];
      if (NIN > 1) oy += cd * a.stride[2][d];
      outer = q;
    }
    if (VEC > 1) {
      VT vx = *reinterpret_cast<const VT*>(x + ox), vy, out;
      if (NIN > 1) vy = *reinterpret_cast<const VT*>(y + oy);
#pragma unroll
      for (int e = 0; e < VEC; e++) {
        if (NIN > 1) out.v[e] = Conv<T>::from(F::template apply<A>((A)to_float(vx.v[e]), (A)to_float(vy.v[e])));
        else out.v[e] = Conv<T>::from(F::template apply<A>((A)to_float(vx.v[e]), (A)to_float(vx.v[e])));
      }
      *reinterpret_cast<VT*>(z + oz) = out;
    } else {
      A vx = (A)to_float(x[ox]);
      A vy = NIN > 1 ? (A)to_float(y[oy]) : vx;
      z[oz] = Conv<T>::from(F::template apply<A>(vx, vy));
    }
  }
}

// adapters so that ew_nd can run unary functors through the two-argument call
template <int K> struct UnaryAs2 { template <typename A> static __device__ __forceinline__ A apply(A a, A) { return Unary<K>::template apply<A>(a); } };

// ---- generic kernel (own shapes, run-time dtypes) ------------------------------------------------------
__device__ __forceinline__ double load_any(const void* p, int dt, LongType off) {
  switch (dt) {
    case FLOAT32: return ((const float*)p)[off];
    case DOUBLE: return ((const double*)p)[off];
    case HALF: return to_float(((const f16_t*)p)[off]);
    case BFLOAT16: return to_float(((const bf16_t*)p)[off]);
    case INT32: return ((const int*)p)[off];
    case INT64: return (double)((const LongType*)p)[off];
    case BOOL: return ((const unsigned char*)p)[off];
    default: return 0.0;
  }
}
__device__ __forceinline__ void store_any(void* p, int dt, LongType off, double v) {
  switch (dt) {
    case FLOAT32: ((float*)p)[off] = (float)v; break;
    case DOUBLE: ((double*)p)[off] = v; break;
    case HALF: ((f16_t*)p)[off] = Conv<f16_t>::from((float)v); break;
    case BFLOAT16: ((bf16_t*)p)[off] = Conv<bf16_t>::from((float)v); break;
    case INT32: ((int*)p)[off] = (int)v; break;
    case INT64: ((LongType*)p)[off] = (LongType)v; break;
    case BOOL: ((unsigned char*)p)[off] = v != 0.0; break;
    default: break;
  }
}
// rounding through the output storage type, applied to operands before the arithmetic as the reference's
// sd_add<X,Y,Z> family casts both operands to Z first
__device__ __forceinline__ float round_as(float v, int dt) {
  if (dt == HALF) return to_float(Conv<f16_t>::from(v));
  if (dt == BFLOAT16) return to_float(Conv<bf16_t>::from(v));
  return v;
}

template <typename F, int NIN>
__global__ __launch_bounds__(EW_BLOCK) void ew_generic(DevShape sz, DevShape sx, DevShape sy, int zdt, int xdt, int ydt,
                                                       void* z, const void* x, const void* y, LongType n) {
  const LongType step = (LongType)gridDim.x * EW_BLOCK;
  for (LongType i = (LongType)blockIdx.x * EW_BLOCK + threadIdx.x; i < n; i += step) {
    LongType oz = walk<LongType>(sz, i), ox = walk<LongType>(sx, i);
    double a = load_any(x, xdt, ox), b = a;
    if (NIN > 1) b = load_any(y, ydt, walk<LongType>(sy, i));
    if (zdt == DOUBLE) store_any(z, zdt, oz, F::template apply<double>(a, b));
    else store_any(z, zdt, oz, F::template apply<float>(round_as((float)a, zdt), round_as((float)b, zdt)));
  }
}

// ---- launch helpers ------------------------------------------------------------------------------------
static int gridFor(LongType work, int perBlock) {
  LongType blocks = (work + perBlock - 1) / perBlock;
  // 256 CUs; a few resident blocks per CU keep enough loads in flight while the loop amortises launch cost
  const LongType cap = 256 * 16;
  if (blocks > cap) blocks = cap;
  if (blocks < 1) blocks = 1;
  return (int)blocks;
}
// does a kernel's total traffic exceed what the last-level cache (256 MB) can usefully hold
static bool streamsPastCache(size_t bytes) { return bytes > (size_t)288 << 20; }
static bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

template <typename F2, typename T, int NIN>
static void launchNd(hipStream_t s, const EwPlan& p, const T* x, const T* y, T* z) {
  constexpr int V = 16 / sizeof(T);
  NdArgs a;
  a.rank = p.rank;
  for (int d = 0; d < p.rank; d++) {
    a.shape[d] = p.shape[d];
    for (int o = 0; o < 3; o++) a.stride[o][d] = p.stride[o][d];
  }
  const LongType inner = p.shape[p.rank - 1];
  bool vec = inner % V == 0 && aligned16(x) && aligned16(z) && (NIN < 2 || aligned16(y));
  for (int o = 0; o <= NIN && vec; o++) {
    if (p.stride[o][p.rank - 1] != 1) vec = false;
    for (int d = 0; d < p.rank - 1; d++) if (p.stride[o][d] % V != 0) vec = false;
  }
  if (vec) {
    LongType cpr = inner / V, total = p.length / V;
    if (p.index32) hipLaunchKernelGGL((ew_nd<F2, T, NIN, V, unsigned>), dim3(gridFor(total, EW_BLOCK)), dim3(EW_BLOCK), 0, s, a, x, y, z, (unsigned)cpr, (unsigned)total);
    else hipLaunchKernelGGL((ew_nd<F2, T, NIN, V, unsigned long long>), dim3(gridFor(total, EW_BLOCK)), dim3(EW_BLOCK), 0, s, a, x, y, z, (unsigned long long)cpr, (unsigned long long)total);
  } else {
    LongType cpr = inner, total = p.length;
    if (p.index32) hipLaunchKernelGGL((ew_nd<F2, T, NIN, 1, unsigned>), dim3(gridFor(total, EW_BLOCK)), dim3(EW_BLOCK), 0, s, a, x, y, z, (unsigned)cpr, (unsigned)total);
    else hipLaunchKernelGGL((ew_nd<F2, T, NIN, 1, unsigned long long>), dim3(gridFor(total, EW_BLOCK)), dim3(EW_BLOCK), 0, s, a, x, y, z, (unsigned long long)cpr, (unsigned long long)total);
  }
}

template <int K, typename T>
static void unaryTyped(hipStream_t s, const EwPlan& p, const void* x, void* z) {
  const T* xt = (const T*)x;
  T* zt = (T*)z;
  if (p.contiguous && aligned16(x) && aligned16(z)) {
    constexpr int V = 16 / sizeof(T);
    const unsigned grid = (unsigned)((p.length / V + EW_BLOCK) / EW_BLOCK);
    if (streamsPastCache(2 * sizeof(T) * (size_t)p.length)) hipLaunchKernelGGL((unary_contig<Unary<K>, T, true>), dim3(grid), dim3(EW_BLOCK), 0, s, xt, zt, p.length);
    else hipLaunchKernelGGL((unary_contig<Unary<K>, T, false>), dim3(grid), dim3(EW_BLOCK), 0, s, xt, zt, p.length);
  } else {
    launchNd<UnaryAs2<K>, T, 1>(s, p, xt, (const T*)nullptr, zt);
  }
}
template <int K>
static void unaryKind(hipStream_t s, DataType xdt, DataType zdt, const void* x, void* z, const EwPlan& p) {
  if (p.sameShape && xdt == zdt && p.rank >= 1) {
    switch (xdt) {
      case FLOAT32: return unaryTyped<K, float>(s, p, x, z);
      case DOUBLE: return unaryTyped<K, double>(s, p, x, z);
      case HALF: return unaryTyped<K, f16_t>(s, p, x, z);
      case BFLOAT16: return unaryTyped<K, bf16_t>(s, p, x, z);
      default: break;
    }
  }
  hipLaunchKernelGGL((ew_generic<UnaryAs2<K>, 1>), dim3(gridFor(p.length, EW_BLOCK)), dim3(EW_BLOCK), 0, s, p.own[0], p.own[1], p.own[1], (int)zdt, (int)xdt, (int)xdt, z, x, x, p.length);
}

void launchUnary(hipStream_t s, UnaryKind k, DataType xdt, DataType zdt, const void* x, void* z, const EwPlan& p) {
  if (p.length == 0) return;
  switch (k) {
#define CASE(K) case K: unaryKind<K>(s, xdt, zdt, x, z, p); break;
    CASE(U_COS) CASE(U_EXP) CASE(U_LOG) CASE(U_SIGMOID) CASE(U_SIN) CASE(U_SOFTPLUS) CASE(U_TANH) CASE(U_SWISH)
    CASE(U_ERF) CASE(U_GELU) CASE(U_PRECISE_GELU) CASE(U_SQRT) CASE(U_RSQRT) CASE(U_ABS) CASE(U_NEG) CASE(U_SQUARE)
    CASE(U_RECIPROCAL) CASE(U_IDENTITY) CASE(U_ONE_MINUS) CASE(U_CUBE)
#undef CASE
    default: ND4J_THROW("launchUnary: unknown op kind");
  }
  HIP_CHECK(hipGetLastError());
}

template <int K, typename T>
static void pairwiseTyped(hipStream_t s, const EwPlan& p, const void* x, const void* y, void* z) {
  const T* xt = (const T*)x; const T* yt = (const T*)y; T* zt = (T*)z;
  if (p.contiguous && aligned16(x) && aligned16(y) && aligned16(z)) {
    constexpr int V = 16 / sizeof(T);
    const unsigned grid = (unsigned)((p.length / V + EW_BLOCK) / EW_BLOCK);
    if (streamsPastCache(3 * sizeof(T) * (size_t)p.length)) hipLaunchKernelGGL((pairwise_contig<Pairwise<K>, T, true>), dim3(grid), dim3(EW_BLOCK), 0, s, xt, yt, zt, p.length);
    else hipLaunchKernelGGL((pairwise_contig<Pairwise<K>, T, false>), dim3(grid), dim3(EW_BLOCK), 0, s, xt, yt, zt, p.length);
  } else {
    launchNd<Pairwise<K>, T, 2>(s, p, xt, yt, zt);
  }
}
template <int K>
static void pairwiseKind(hipStream_t s, DataType xdt, DataType ydt, DataType zdt, const void* x, const void* y, void* z,
                         const EwPlan& p) {
  if (p.sameShape && xdt == zdt && ydt == zdt && p.rank >= 1) {
    switch (zdt) {
      case FLOAT32: return pairwiseTyped<K, float>(s, p, x, y, z);
      case DOUBLE: return pairwiseTyped<K, double>(s, p, x, y, z);
      case HALF: return pairwiseTyped<K, f16_t>(s, p, x, y, z);
      case BFLOAT16: return pairwiseTyped<K, bf16_t>(s, p, x, y, z);
      default: break;
    }
  }
  hipLaunchKernelGGL((ew_generic<Pairwise<K>, 2>), dim3(gridFor(p.length, EW_BLOCK)), dim3(EW_BLOCK), 0, s, p.own[0], p.own[1], p.own[2], (int)zdt, (int)xdt, (int)ydt, z, x, y, p.length);
}

void launchPairwise(hipStream_t s, PairwiseKind k, DataType xdt, DataType ydt, DataType zdt, const void* x,
                    const void* y, void* z, const EwPlan& p) {
  if (p.length == 0) return;
  switch (k) {
#define CASE(K) case K: pairwiseKind<K>(s, xdt, ydt, zdt, x, y, z, p); break;
    CASE(P_ADD) CASE(P_COPY) CASE(P_DIV) CASE(P_MUL) CASE(P_RSUB) CASE(P_SUB) CASE(P_MAX) CASE(P_MIN) CASE(P_RDIV)
    CASE(P_SQSUB)
#undef CASE
    default: ND4J_THROW("launchPairwise: unknown op kind");
  }
  HIP_CHECK(hipGetLastError());
}

// ---- broadcast of a vector along the last axis / scalar ops ----------------------------------------------
template <typename F, typename T>
__global__ __launch_bounds__(EW_BLOCK) void row_broadcast(const T* __restrict__ x, const T* __restrict__ v,
                                                          T* __restrict__ z, LongType rows, LongType cols) {
  using A = typename Conv<T>::acc;
  const LongType n = rows * cols;
  const LongType step = (LongType)gridDim.x * EW_BLOCK;
  for (LongType i = (LongType)blockIdx.x * EW_BLOCK + threadIdx.x; i < n; i += step) {
    LongType c = i % cols;
    z[i] = Conv<T>::from(F::template apply<A>((A)to_float(x[i]), (A)to_float(v[c])));
  }
}
template <typename F, typename T>
__global__ __launch_bounds__(EW_BLOCK) void row_broadcast_vec(const T* __restrict__ x, const T* __restrict__ v,
                                                              T* __restrict__ z, LongType rows, LongType colVecs) {
  constexpr int V = 16 / sizeof(T);
  using VT = Vec<T, V>;
  using A = typename Conv<T>::acc;
  const LongType n = rows * colVecs;
  const LongType step = (LongType)gridDim.x * EW_BLOCK;
  const VT* xv = reinterpret_cast<const VT*>(x);
  const VT* vv = reinterpret_cast<const VT*>(v);
  VT* zv = reinterpret_cast<VT*>(z);
  for (LongType i = (LongType)blockIdx.x * EW_BLOCK + threadIdx.x; i < n; i += step) {
    VT a = xv[i], b = vv[i % colVecs], out;
#pragma unroll
    for (int e = 0; e < V; e++) out.v[e] = Conv<T>::from(F::template apply<A>((A)to_float(a.v[e]), (A)to_float(b.v[e])));
    zv[i] = out;
  }
}
template <int K, typename T>
static void rowBroadcastTyped(hipStream_t s, const void* x, const void* v, void* z, LongType rows, LongType cols) {
  constexpr int V = 16 / sizeof(T);
  if (cols % V == 0 && aligned16(x) && aligned16(v) && aligned16(z))
    hipLaunchKernelGGL((row_broadcast_vec<Pairwise<K>, T>), dim3(gridFor(rows * cols / V, EW_BLOCK)), dim3(EW_BLOCK), 0, s, (const T*)x, (const T*)v, (T*)z, rows, cols / V);
  else
    hipLaunchKernelGGL((row_broadcast<Pairwise<K>, T>), dim3(gridFor(rows * cols, EW_BLOCK)), dim3(EW_BLOCK), 0, s, (const T*)x, (const T*)v, (T*)z, rows, cols);
}
template <int K>
static void rowBroadcastKind(hipStream_t s, DataType dt, const void* x, const void* v, void* z, LongType rows, LongType cols) {
  switch (dt) {
    case FLOAT32: return rowBroadcastTyped<K, float>(s, x, v, z, rows, cols);
    case DOUBLE: return rowBroadcastTyped<K, double>(s, x, v, z, rows, cols);
    case HALF: return rowBroadcastTyped<K, f16_t>(s, x, v, z, rows, cols);
    case BFLOAT16: return rowBroadcastTyped<K, bf16_t>(s, x, v, z, rows, cols);
    default: ND4J_THROW("row broadcast: unsupported dtype");
  }
}
void launchRowBroadcast(hipStream_t s, PairwiseKind k, DataType dt, const void* x, const void* v, void* z,
                        LongType rows, LongType cols) {
  if (rows * cols == 0) return;
  switch (k) {
    case P_ADD: rowBroadcastKind<P_ADD>(s, dt, x, v, z, rows, cols); break;
    case P_SUB: rowBroadcastKind<P_SUB>(s, dt, x, v, z, rows, cols); break;
    case P_MUL: rowBroadcastKind<P_MUL>(s, dt, x, v, z, rows, cols); break;
    case P_DIV: rowBroadcastKind<P_DIV>(s, dt, x, v, z, rows, cols); break;
    default: ND4J_THROW("row broadcast: unsupported op");
  }
  HIP_CHECK(hipGetLastError());
}

template <typename F, typename T>
__global__ __launch_bounds__(EW_BLOCK) void scalar_nd(NdArgs a, const T* __restrict__ x, T* __restrict__ z,
                                                      typename Conv<T>::acc sc, LongType n) {
  using A = typename Conv<T>::acc;
  const LongType step = (LongType)gridDim.x * EW_BLOCK;
  for (LongType i = (LongType)blockIdx.x * EW_BLOCK + threadIdx.x; i < n; i += step) {
    LongType idx = i, oz = 0, ox = 0;
#pragma unroll 1
    for (int d = a.rank - 1; d >= 0; d--) {
      LongType q = idx / a.shape[d], c = idx - q * a.shape[d];
      oz += c * a.stride[0][d]; ox += c * a.stride[1][d]; idx = q;
    }
    z[oz] = Conv<T>::from(F::template apply<A>((A)to_float(x[ox]), sc));
  }
}
template <int K, typename T>
static void scalarTyped(hipStream_t s, const void* x, double sc, void* z, const EwPlan& p) {
  NdArgs a;
  a.rank = p.rank;
  for (int d = 0; d < p.rank; d++) { a.shape[d] = p.shape[d]; for (int o = 0; o < 3; o++) a.stride[o][d] = p.stride[o][d]; }
  using A = typename Conv<T>::acc;
  A scv = (A)sc;
  hipLaunchKernelGGL((scalar_nd<Pairwise<K>, T>), dim3(gridFor(p.length, EW_BLOCK)), dim3(EW_BLOCK), 0, s, a, (const T*)x, (T*)z, scv, p.length);
}
template <int K>
static void scalarKind(hipStream_t s, DataType dt, const void* x, double sc, void* z, const EwPlan& p) {
  switch (dt) {
    case FLOAT32: return scalarTyped<K, float>(s, x, sc, z, p);
    case DOUBLE: return scalarTyped<K, double>(s, x, sc, z, p);
    case HALF: return scalarTyped<K, f16_t>(s, x, sc, z, p);
    case BFLOAT16: return scalarTyped<K, bf16_t>(s, x, sc, z, p);
    default: ND4J_THROW("scalar op: unsupported dtype");
  }
}
void launchScalarOp(hipStream_t s, PairwiseKind k, DataType dt, const void* x, double scalar, void* z, const EwPlan& p) {
  if (p.length == 0) return;
  ND4J_REQUIRE(p.sameShape && p.rank >= 1, "scalar op: operands must share a shape");
  switch (k) {
    case P_ADD: scalarKind<P_ADD>(s, dt, x, scalar, z, p); break;
    case P_SUB: scalarKind<P_SUB>(s, dt, x, scalar, z, p); break;
    case P_MUL: scalarKind<P_MUL>(s, dt, x, scalar, z, p); break;
    case P_DIV: scalarKind<P_DIV>(s, dt, x, scalar, z, p); break;
    case P_RSUB: scalarKind<P_RSUB>(s, dt, x, scalar, z, p); break;
    case P_RDIV: scalarKind<P_RDIV>(s, dt, x, scalar, z, p); break;
    case P_MAX: scalarKind<P_MAX>(s, dt, x, scalar, z, p); break;
    case P_MIN: scalarKind<P_MIN>(s, dt, x, scalar, z, p); break;
    case P_COPY: scalarKind<P_COPY>(s, dt, x, scalar, z, p); break;
    default: ND4J_THROW("scalar op: unsupported op");
  }
  HIP_CHECK(hipGetLastError());
}

// ---- gather rows / fill ------------------------------------------------------------------------------------
template <typename T, typename IT>
__global__ __launch_bounds__(EW_BLOCK) void gather_rows(const T* __restrict__ table, const IT* __restrict__ idx,
                                                        T* __restrict__ z, LongType nIdx, LongType rowLen, LongType tableRows) {
  const LongType n = nIdx * rowLen;
  const LongType step = (LongType)gridDim.x * EW_BLOCK;
  for (LongType i = (LongType)blockIdx.x * EW_BLOCK + threadIdx.x; i < n; i += step) {
    LongType r = i / rowLen, c = i - r * rowLen;
    LongType src = (LongType)idx[r];
    if (src < 0) src += tableRows;
    // out-of-range ids are clamped so that a bad id cannot fault the device; the host validates ids it can see
    src = src < 0 ? 0 : (src >= tableRows ? tableRows - 1 : src);
    z[i] = table[src * rowLen + c];
  }
}
void launchGatherRows(hipStream_t s, DataType dt, DataType idxDt, const void* table, const void* idx, void* z,
                      LongType nIdx, LongType rowLen, LongType tableRows) {
  if (nIdx * rowLen == 0) return;
  ND4J_REQUIRE(idxDt == INT32 || idxDt == INT64, "gather: indices must be INT32 or INT64");
  dim3 g(gridFor(nIdx * rowLen, EW_BLOCK)), b(EW_BLOCK);
#define GATHER(T)                                                                                                         \
  if (idxDt == INT32) hipLaunchKernelGGL((gather_rows<T, int>), g, b, 0, s, (const T*)table, (const int*)idx, (T*)z, nIdx, rowLen, tableRows); \
  else hipLaunchKernelGGL((gather_rows<T, LongType>), g, b, 0, s, (const T*)table, (const LongType*)idx, (T*)z, nIdx, rowLen, tableRows);
  switch (sizeOf(dt)) {
    case 2: GATHER(unsigned short) break;
    case 4: GATHER(unsigned) break;
    case 8: GATHER(unsigned long long) break;
    default: ND4J_THROW("gather: unsupported element size");
  }
#undef GATHER
  HIP_CHECK(hipGetLastError());
}

__global__ __launch_bounds__(EW_BLOCK) void fill_bytes(unsigned char* p, unsigned char v, size_t n) {
  const size_t step = (size_t)gridDim.x * EW_BLOCK;
  for (size_t i = (size_t)blockIdx.x * EW_BLOCK + threadIdx.x; i < n; i += step) p[i] = v;
}
void launchFill(hipStream_t s, void* p, int byteValue, size_t bytes) {
  if (bytes == 0) return;
  hipLaunchKernelGGL(fill_bytes, dim3(gridFor((LongType)bytes, EW_BLOCK)), dim3(EW_BLOCK), 0, s, (unsigned char*)p, (unsigned char)byteValue, bytes);
  HIP_CHECK(hipGetLastError());
}

}  // namespace nd4jhip
