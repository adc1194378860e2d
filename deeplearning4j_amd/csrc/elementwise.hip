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
#include "anyio.h"
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

// applyLow is what the contiguous kernel calls for 16-bit arrays: the same function where a cheaper evaluation only moves
// the fp32 value by a few 1e-7 relative, far below half a unit of a bf16 / fp16 result (those launches are bound by
// instruction issue, not by memory: twice the elements per byte).
template <int K> struct Unary;
#define UNARY_LOW(K, EXPR, LOWEXPR) \
  template <> struct Unary<K> { \
    template <typename A> static __device__ __forceinline__ A apply(A x) { return EXPR; } \
    template <typename A> static __device__ __forceinline__ A applyLow(A x) { return LOWEXPR; } }
#define UNARY(K, EXPR) UNARY_LOW(K, EXPR, EXPR)
// 1 / (1 + e^-x) with the exponential as one v_exp_f32 of x * log2(e)
__device__ __forceinline__ float d_sigmoid_low(float x) { return fast_rcp(1.f + __builtin_amdgcn_exp2f(x * -1.44269502162933349609375f)); }
__device__ __forceinline__ double d_sigmoid_low(double x) { return 1.0 / (1.0 + exp(-x)); }
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
UNARY_LOW(U_SIGMOID, d_sigmoid<A>(x), d_sigmoid_low(x));       // ops.h:200
UNARY(U_SIN, d_sin(x));                                        // ops.h:198
UNARY(U_SOFTPLUS, d_log((A)1 + fast_exp(x)));                  // templatemath.h:272-274
UNARY(U_TANH, d_tanh(x));                                      // ops.h:199
UNARY_LOW(U_SWISH, x * d_sigmoid<A>(x), x * d_sigmoid_low(x)); // ops.h:988-990
UNARY(U_ERF, d_erf(x));                                        // ops.h:361
__device__ __forceinline__ double gelu_full(double x) { return x * d_sigmoid<double>(1.702f * x); }
__device__ __forceinline__ double gelu_low(double x) { return x * d_sigmoid_low(1.702f * x); }
UNARY_LOW(U_GELU, gelu_full(x), gelu_low(x));   // ops.h:1010-1012; the float forms live in device.h, shared with the GEMM epilogue
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

// ---- the long tail of the op tables: op picked at run time inside one kernel per dtype ------------------------
// Formulas restate ops/ops.h and math/templatemath.h of the reference (line numbers beside each case).  A = float
// for the half/bfloat16/float flavours, double for double.
template <typename A> struct Tm;
template <> struct Tm<float> {
  static __device__ __forceinline__ float exp_(float x) { return expf(x); }
  static __device__ __forceinline__ float log_(float x) { return logf(x); }
  static __device__ __forceinline__ float cosh_(float x) { return coshf(x); }
  static __device__ __forceinline__ float sinh_(float x) { return sinhf(x); }
  static __device__ __forceinline__ float tan_(float x) { return tanf(x); }
  static __device__ __forceinline__ float acos_(float x) { return acosf(x); }
  static __device__ __forceinline__ float asin_(float x) { return asinf(x); }
  static __device__ __forceinline__ float atan_(float x) { return atanf(x); }
  static __device__ __forceinline__ float acosh_(float x) { return acoshf(x); }
  static __device__ __forceinline__ float asinh_(float x) { return asinhf(x); }
  static __device__ __forceinline__ float atanh_(float x) { return atanhf(x); }
  static __device__ __forceinline__ float erfc_(float x) { return erfcf(x); }
  static __device__ __forceinline__ float rint_(float x) { return rintf(x); }
  static __device__ __forceinline__ float round_(float x) { return roundf(x); }
  static __device__ __forceinline__ float ceil_(float x) { return ceilf(x); }
  static __device__ __forceinline__ float floor_(float x) { return floorf(x); }
  static __device__ __forceinline__ float pow_(float a, float b) { return powf(a, b); }
  static __device__ __forceinline__ float fmod_(float a, float b) { return fmodf(a, b); }
  static __device__ __forceinline__ float remainder_(float a, float b) { return remainderf(a, b); }
  static __device__ __forceinline__ float atan2_(float a, float b) { return atan2f(a, b); }
  static __device__ __forceinline__ float gamma_(float x) { return tgammaf(x); }
};
template <> struct Tm<double> {
  static __device__ __forceinline__ double exp_(double x) { return exp(x); }
  static __device__ __forceinline__ double log_(double x) { return log(x); }
  static __device__ __forceinline__ double cosh_(double x) { return cosh(x); }
  static __device__ __forceinline__ double sinh_(double x) { return sinh(x); }
  static __device__ __forceinline__ double tan_(double x) { return tan(x); }
  static __device__ __forceinline__ double acos_(double x) { return acos(x); }
  static __device__ __forceinline__ double asin_(double x) { return asin(x); }
  static __device__ __forceinline__ double atan_(double x) { return atan(x); }
  static __device__ __forceinline__ double acosh_(double x) { return acosh(x); }
  static __device__ __forceinline__ double asinh_(double x) { return asinh(x); }
  static __device__ __forceinline__ double atanh_(double x) { return atanh(x); }
  static __device__ __forceinline__ double erfc_(double x) { return erfc(x); }
  static __device__ __forceinline__ double rint_(double x) { return rint(x); }
  static __device__ __forceinline__ double round_(double x) { return round(x); }
  static __device__ __forceinline__ double ceil_(double x) { return ceil(x); }
  static __device__ __forceinline__ double floor_(double x) { return floor(x); }
  static __device__ __forceinline__ double pow_(double a, double b) { return pow(a, b); }
  static __device__ __forceinline__ double fmod_(double a, double b) { return fmod(a, b); }
  static __device__ __forceinline__ double remainder_(double a, double b) { return remainder(a, b); }
  static __device__ __forceinline__ double atan2_(double a, double b) { return atan2(a, b); }
  static __device__ __forceinline__ double gamma_(double x) { return tgamma(x); }
};
// 1 / (1 + e^-x) with the library exponential: derivatives subtract it from one, so it keeps full precision
template <typename A> __device__ __forceinline__ A exact_sigmoid(A x) { return (A)1 / ((A)1 + Tm<A>::exp_(-x)); }
template <typename A> __device__ __forceinline__ A sgn_(A x) { return x < (A)0 ? (A)-1 : x > (A)0 ? (A)1 : (A)0; }   // templatemath.h:359-362

template <typename A>
__device__ __forceinline__ A unary_tail(int k, A x) {
  using M = Tm<A>;
  const A one = (A)1;
  switch (k) {
    case U_TANH_D: { A t = d_tanh(x); return one - t * t; }                                   // templatemath.h:335-339
    case U_SIGMOID_D: { A s = exact_sigmoid(x); return s * (one - s); }                       // templatemath.h:343-347
    case U_SOFTSIGN_D: { A y = one + d_abs(x); return one / (y * y); }                        // templatemath.h:351-355
    case U_TAN_D: { A c = d_cos(x); return one / (c * c); }                                   // ops.h:169
    case U_SELU_D: return x > (A)0 ? (A)1.0507009873554804934193349852946                     // ops.h:966-970
                                   : (A)1.6732632423543772848170429916717 * (A)1.0507009873554804934193349852946 * M::exp_(x);
    case U_RATIONAL_TANH_D: {                                                                 // ops.h:1076-1086
      A dis = ((A)2 / (A)3) * x, d2 = dis * dis;
      A a = one + d_abs(dis) + d2 + (A)1.41645f * d2 * d2;
      A t = (one + sgn_(dis) * ((A)2 * dis + (A)4 * (A)1.41645f * d2 * dis)) / (a * a);
      return (A)1.7159f * ((A)2 / (A)3) * t;
    }
    case U_RECTIFIED_TANH_D: { if (!(x > (A)0)) return (A)0; A t = d_tanh(x); return one - t * t; }   // ops.h:72-75
    case U_SWISH_D: { A ex = M::exp_(x), d = ex + one; return (ex * (x + ex + one)) / (d * d); }      // ops.h:993-996
    case U_ACOSH_D: return one / (d_sqrt(x - one) * d_sqrt(x + one));                          // ops.h:159-160
    case U_ASINH_D: return one / d_sqrt(x * x + one);                                          // ops.h:155-156
    case U_SINH_D: return M::cosh_(x);                                                         // ops.h:1048
    case U_LOG_SIGMOID_D: return one / (M::exp_(x) + one);                                     // ops.h:1042-1045
    case U_SPECIAL_D: return x * (one - x);                                                    // ops.h:1167
    case U_CUBE_D: return (A)3 * x * x;                                                        // ops.h:1166
    case U_ACOS: return M::acos_(x);                                                           // ops.h:364
    case U_ASIN: return M::asin_(x);                                                           // ops.h:363
    case U_ATAN: return M::atan_(x);                                                           // ops.h:365
    case U_HARD_TANH: return x < (A)-1 ? (A)-1 : x > one ? one : x;                            // ops.h:67-70
    case U_SOFTSIGN: return x / (one + d_abs(x));                                              // templatemath.h:302-306
    case U_HARD_SIGMOID: { A v = (A)0.2f * x + (A)0.5f; v = v > (A)0 ? v : (A)0; return v < one ? v : one; }   // ops.h:973-976
    case U_RATIONAL_TANH: {                                                                    // ops.h:1065-1074
      A dis = ((A)2 / (A)3) * x, d2 = dis * dis;
      A t = sgn_(dis) * (one - one / (one + d_abs(dis) + d2 + (A)1.41645f * d2 * d2));
      return (A)1.7159f * t;
    }
    case U_RECTIFIED_TANH: { A t = d_tanh(x); return t > (A)0 ? t : (A)0; }                    // ops.h:1093-1095
    case U_SINH: return M::sinh_(x);                                                           // ops.h:369
    case U_COSH: return M::cosh_(x);                                                           // ops.h:370
    case U_TAN: return M::tan_(x);                                                             // ops.h:371
    case U_SELU: return x > (A)0 ? (A)1.0507009873554804934193349852946 * x                    // ops.h:978-982
                                 : (A)1.0507009873554804934193349852946 *
                                       ((A)1.6732632423543772848170429916717 * M::exp_(x) - (A)1.6732632423543772848170429916717);
    case U_LOG1P: return M::log_(one + x);                                                     // ops.h:375
    case U_ACOSH: return M::acosh_(x);                                                         // ops.h:368
    case U_ASINH: return M::asinh_(x);                                                         // ops.h:367
    case U_RINT: return M::rint_(x);                                                           // ops.h:360
    case U_LOG_SIGMOID: return M::log_(exact_sigmoid(x));                                      // ops.h:1038-1040
    case U_ERFC: return M::erfc_(x);                                                           // ops.h:362
    case U_EXPM1: return M::exp_(x) - one;                                                     // ops.h:378
    case U_ATANH: return M::atanh_(x);                                                         // ops.h:366
    case U_GELU_D: {                                                                           // ops.h:1020-1025
      A x17 = (A)1.702f * x, ep = M::exp_(x17), o = one + ep;
      return (ep * (o + x17)) / (o * o);
    }
    case U_PRECISE_GELU_D: {                                                                   // ops.h:1027-1036
      A x79 = (A)0.797885 * x, t1 = (A)0.0356774 * x, x03 = t1 * t1 * t1;
      A x39 = (A)0.398942 * x, t2 = (A)0.0535161 * x, x05 = t2 * t2 * t2;
      A scz = one / M::cosh_(x79 + x03);
      return (A)0.5 + (x39 + x05) * (scz * scz) + (A)0.5 * d_tanh(x79 + x03);
    }
    case U_MISH: return x * d_tanh(M::log_(one + M::exp_(x)));                                 // ops.h:999-1001
    case U_MISH_D: {                                                                           // ops.h:1003-1008
      A ex = M::exp_(x), e2x = ex * ex, e3x = ex * ex * ex, d = (A)2 * ex + e2x + (A)2;
      return (ex * ((A)4 * (x + one) + (A)4 * e2x + e3x + ex * ((A)4 * x + (A)6))) / (d * d);
    }
    case U_ONES: return one;                                                                   // ops.h:481
    case U_ROUND: return M::round_(x);                                                         // ops.h:359
    case U_TIMES_ONE_MINUS: return x * (one - x);                                              // ops.h:1165
    case U_CEIL: return M::ceil_(x);                                                           // ops.h:193
    case U_FLOOR: return M::floor_(x);                                                         // ops.h:196
    // ops.h:217-219 through op_macros_unary.h:109-113: the sign expression is the CONDITION, so every non-zero number gives 1
    case U_SIGN_REF: return ((x > (A)0) - (x < (A)0)) != 0 ? one : -one;
    case U_STABILIZE_FP16: return x <= (A)0 ? (A)6.103515625e-05 : x;                          // ops.h:381-384 (HALF's smallest normal)
    // TransformBool (ops.h:1140-1163,1927-1933): 1 where the predicate holds
    case U_IS_INF: return (x == x && (x - x) != (x - x)) ? one : (A)0;
    case U_IS_NAN: return x != x ? one : (A)0;
    case U_IS_FINITE: return (x - x) == (x - x) ? one : (A)0;
    case U_IS_INF_OR_NAN: return (x - x) == (x - x) ? (A)0 : one;
    case U_IS_POSITIVE: return x > (A)0 ? one : (A)0;
    case U_IS_NEGATIVE: return x < (A)0 ? one : (A)0;
    case U_NOT: return x == (A)0 ? one : (A)0;
    default: return x;
  }
}

// |a - b| / (|a| + |b|), 0 for two zeros (templatemath.h:1144-1153)
template <typename A> __device__ __forceinline__ A rel_err(A a, A b) { return (a == (A)0 && b == (A)0) ? (A)0 : d_abs(a - b) / (d_abs(a) + d_abs(b)); }
// Regularised lower incomplete gamma function as the reference sums it (templatemath.h:963-984): x^a e^-x / Gamma(a) times
// the series sum x^i / (a (a+1) .. (a+i)), cut off when the running denominator passes 1e12 (whatever x is), 0 for a <= 1e-6
template <typename A>
__device__ __forceinline__ A igamma_(A a, A x) {
  if (a <= (A)0.000001) return (A)0;
  const A aim = Tm<A>::pow_(x, a) / (Tm<A>::exp_(x) * Tm<A>::gamma_(a));
  A sum = (A)0, denom = (A)1, xi = (A)1;
  for (int i = 0; (A)1 / denom > (A)1.0e-12 && i < 4096; i++) {
    denom *= a + (A)i;
    sum += xi / denom;
    xi *= x;
  }
  return aim * sum;
}

// a = element of x, b = element of y or the scalar
template <typename A>
__device__ __forceinline__ A binary_tail(int k, A a, A b) {
  using M = Tm<A>;
  switch (k) {
    case P_POW: return M::pow_(a, b);                                                          // ops.h:165
    case P_REMAINDER: return M::remainder_(a, b);                                              // ops.h:228
    case P_FMOD: return M::fmod_(a, b);                                                        // ops.h:229
    case P_ATAN2: return M::atan2_(a, b);                                                      // ops.h:79, templatemath.h:321-324
    case P_TRUNCATE_DIV: { int ib = (int)b; return ib == 0 ? (A)0 : (A)((int)a / ib); }        // ops.h:240-245 (a zero divisor traps there)
    case P_FLOOR_DIV: return (A)floor((double)a / (double)b);                                  // op_macros_special.h:87-93
    case P_FLOOR_MOD: {                                                                        // ops.h:260-267
      A m = M::fmod_(a, b);
      return ((a < (A)0) == (b < (A)0)) ? m : M::fmod_(m + b, b);
    }
    case P_REVERSE_MOD: { int ia = (int)a; return ia == 0 ? (A)0 : (A)((int)b % ia); }         // ops.h:1747-1752
    case P_SAFE_DIVIDE: case P_DIVIDE_NO_NAN: return b == (A)0 ? (A)0 : a / b;                 // ops.h:232-233
    case P_MOD: return a - M::floor_(a / b) * b;                                               // ops.h:1708-1715
    case P_LOGICAL_OR: return (A)((int)a | (int)b);                                            // ops.h:2423-2428
    case P_LOGICAL_XOR: return (A)(((int)a | (int)b) & ~((int)a & (int)b));                    // ops.h:2407-2412
    case P_LOGICAL_NOT: return (A)(!((int)a && (int)b));                                       // ops.h:2399-2404
    case P_LOGICAL_AND: return (A)((int)a & (int)b);                                           // ops.h:2415-2420
    case P_AMAX: return d_abs(a) > d_abs(b) ? a : b;                                           // ops.h:89-94
    case P_AMIN: return d_abs(a) < d_abs(b) ? a : b;                                           // ops.h:96-101
    case P_TRUNCATE_MOD: { int ib = (int)b; return ib == 0 ? (A)0 : (A)((int)a % ib); }        // ops.h:247-252
    case P_REPLACE_NANS: return a != a ? b : a;                                                // ops.h:582-587
    case P_ELU: return a >= (A)0 ? a : b * (M::exp_(a) - (A)1);                                // templatemath.h:233-240
    case P_ELU_D: return a >= (A)0 ? (A)1 : b * M::exp_(a);                                    // templatemath.h:255-262
    case P_LEAKY_RELU: return a < (A)0 ? b * a : a;                                            // ops.h:1127-1131
    case P_LEAKY_RELU_D: return a >= (A)0 ? (A)1 : b;                                          // ops.h:1133-1138
    case P_LOG_X: return M::log_(a) / M::log_(b);                                              // ops.h:144-149
    case P_RELU: return a < b ? b : a;                                                         // ops.h:1108-1112
    case P_RELU6: { A r = a < b ? b : a; return r < (A)6 ? r : (A)6; }                         // ops.h:1122-1125
    case P_RELU_D: return a > b ? (A)1 : (A)0;                                                 // ops.h:1115-1119
    case P_STEP: return a > b ? (A)1 : (A)0;                                                   // ops.h:347-350
    case P_LSTM_CLIP: return a > b ? b : a < -b ? -b : a;                                      // ops.h:337-345
    case P_SQ_RSUB: { A d = b - a; return d * d; }                                             // op_macros_special.h:820-827
    case P_REVERSE_POW: return M::pow_(b, a);                                                  // ops.h:166
    case P_SXE_LOGITS_SMOOTHER: return a * ((A)1 - b) + (A)0.5f * b;                           // ops.h:352-355
    case P_REL_ERR: return rel_err(a, b);                                                      // ops.h:2208-2213
    case P_POW_DERIV: return b * M::pow_(a, b - (A)1);                                          // ops.h:82-87
    case P_LOG_POISSON: return M::exp_(b) - a * b;                                              // ops.h:2389-2394
    case P_LOG_POISSON_FULL:                                                                    // ops.h:1494-1502 (Stirling term)
      return M::exp_(b) - a * b + (a * M::log_(a) - a + (A)0.5 * M::log_((A)(2.0 * 3.14159265358979323846) * a));
    case P_IGAMMA: return igamma_(a, b);                                                        // ops.h:137, templatemath.h:963-984
    case P_IGAMMAC: return (A)1 - igamma_(a, b);                                                // ops.h:140, templatemath.h:986-991
    case P_EQ: return (A)(a == b);                                                             // ops.h:181-186 (comparison ops)
    case P_NE: return (A)(a != b);
    case P_GT: return (A)(a > b);
    case P_GE: return (A)(a >= b);
    case P_LT: return (A)(a < b);
    case P_LE: return (A)(a <= b);
    default: return a;
  }
}

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

template <typename F, typename T, bool NT, bool NTS>
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
    for (int e = 0; e < V; e++) vals[e] = sizeof(T) == 2 ? F::template applyLow<A>(vals[e]) : F::template apply<A>(vals[e]);
    st_stream<NTS>(reinterpret_cast<RT*>(z) + i, IO::pack(vals));
  }
  // scalar tail (fewer than V elements)
  const LongType tail = nvec * V + i;
  if (tail < n) z[tail] = Conv<T>::from(F::template apply<A>((A)to_float(x[tail])));
}

template <typename F, typename T, bool NT, bool NTS>
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
    st_stream<NTS>(reinterpret_cast<RT*>(z) + i, IO::pack(a));
  }
  const LongType tail = nvec * V + i;
  if (tail < n) z[tail] = Conv<T>::from(F::template apply<A>((A)to_float(x[tail]), (A)to_float(y[tail])));
}
// ---- same-shape strided kernels ------------------------------------------------------------------------
struct NdArgs {
  int rank;                        // >= 1; dim rank-1 is the inner run
  LongType shape[MAX_DEV_RANK];
  LongType stride[3][MAX_DEV_RANK];
  int nts = 0;                     // the vector kernels: the result leaves through non-temporal stores (8 MiB and more)
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
      // an input that repeats along the inner axis (stride 0: a value per row, a scalar) is read once and spread
      VT vx, vy, out;
      if (a.stride[1][a.rank - 1] == 0) {
        const T sx = x[ox];
#pragma unroll
        for (int e = 0; e < VEC; e++) vx.v[e] = sx;
      } else vx = *reinterpret_cast<const VT*>(x + ox);
      if (NIN > 1) {
        if (a.stride[2][a.rank - 1] == 0) {
          const T sy = y[oy];
#pragma unroll
          for (int e = 0; e < VEC; e++) vy.v[e] = sy;
        } else vy = *reinterpret_cast<const VT*>(y + oy);
      }
#pragma unroll
      for (int e = 0; e < VEC; e++) {
        if (NIN > 1) out.v[e] = Conv<T>::from(F::template apply<A>((A)to_float(vx.v[e]), (A)to_float(vy.v[e])));
        else out.v[e] = Conv<T>::from(F::template apply<A>((A)to_float(vx.v[e]), (A)to_float(vx.v[e])));
      }
      store_vec(reinterpret_cast<VT*>(z + oz), out, a.nts != 0);
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

// Tail ops: the same access patterns with the op code as a kernel argument (uniform branch per element).
template <typename T, int NIN>
__global__ __launch_bounds__(EW_BLOCK) void tail_contig(int k, const T* __restrict__ x, const T* __restrict__ y,
                                                        T* __restrict__ z, LongType n) {
  constexpr int V = 16 / sizeof(T);
  using IO = RawIO<T>;
  using RT = typename IO::raw;
  using A = typename Conv<T>::acc;
  const LongType nvec = n / V;
  const LongType i = (LongType)blockIdx.x * EW_BLOCK + threadIdx.x;
  if (i < nvec) {
    A a[V], b[V];
    IO::unpack(*(reinterpret_cast<const RT*>(x) + i), a);
    if (NIN > 1) IO::unpack(*(reinterpret_cast<const RT*>(y) + i), b);
#pragma unroll
    for (int e = 0; e < V; e++) a[e] = NIN > 1 ? binary_tail<A>(k, a[e], b[e]) : unary_tail<A>(k, a[e]);
    *(reinterpret_cast<RT*>(z) + i) = IO::pack(a);
  }
  const LongType tail = nvec * V + i;
  if (tail < n) {
    A a = (A)to_float(x[tail]);
    z[tail] = Conv<T>::from(NIN > 1 ? binary_tail<A>(k, a, (A)to_float(y[tail])) : unary_tail<A>(k, a));
  }
}
// any strides, any float dtypes; hasScalar: the second operand is `scalar`
template <int NIN>
__global__ __launch_bounds__(EW_BLOCK) void tail_generic(int k, DevShape sz, DevShape sx, DevShape sy, int zdt, int xdt, int ydt,
                                                         void* z, const void* x, const void* y, LongType n, double scalar,
                                                         int hasScalar) {
  const LongType step = (LongType)gridDim.x * EW_BLOCK;
  for (LongType i = (LongType)blockIdx.x * EW_BLOCK + threadIdx.x; i < n; i += step) {
    LongType oz = walk<LongType>(sz, i), ox = walk<LongType>(sx, i);
    double a = load_any(x, xdt, ox), b = scalar;
    if (NIN > 1 && !hasScalar) b = load_any(y, ydt, walk<LongType>(sy, i));
    if (zdt == DOUBLE || xdt == DOUBLE || xdt == INT32 || xdt == INT64) {   // predicates on doubles and integers must not see them narrowed
      store_any(z, zdt, oz, NIN > 1 ? binary_tail<double>(k, a, b) : unary_tail<double>(k, a));
    } else {
      float fa = round_as((float)a, zdt), fb = round_as((float)b, zdt);
      store_any(z, zdt, oz, NIN > 1 ? binary_tail<float>(k, fa, fb) : unary_tail<float>(k, fa));
    }
  }
}

// transforms with two parameters; any strides, any float dtypes.  The clip compares in double against the bounds as given
// and stores the bound rounded to the output type (helpers/cpu/clip.cpp:211-219); the other two evaluate in the
// accumulator type of the array (float for 16- and 32-bit arrays).
__device__ __forceinline__ double scalar2_eval(int k, double a, bool inDouble, double s1, double s2) {
  double r;
  if (k == S2_CLIP_BY_VALUE) {
    r = a > s2 ? s2 : (a < s1 ? s1 : a);
  } else if (inDouble) {
    const double cut = (double)3.79297773665f;
    if (k == S2_AFFINE) r = s1 * a + s2;
    else if (k == S2_SCALED_TANH) r = s1 * d_tanh(s2 * a);
    else if (k == S2_STABILIZE) r = a * s1 > cut ? cut / s1 : (a * s1 < -cut ? -cut / s1 : a);
    else if (a >= s1 && a <= s2) r = a;
    else r = floor((s1 == 0.0 && s2 == 1.0 ? 1.0 / (1.0 + exp(-a)) : a) * (s2 - s1)) + s1;
  } else {
    const float fa = (float)a, f1 = (float)s1, f2 = (float)s2, cut = 3.79297773665f;
    if (k == S2_AFFINE) r = f1 * fa + f2;
    else if (k == S2_SCALED_TANH) r = f1 * d_tanh(f2 * fa);
    else if (k == S2_STABILIZE) r = fa * f1 > cut ? cut / f1 : (fa * f1 < -cut ? -cut / f1 : fa);
    else if (fa >= f1 && fa <= f2) r = fa;
    else r = floorf((f1 == 0.f && f2 == 1.f ? 1.f / (1.f + expf(-fa)) : fa) * (f2 - f1)) + f1;
  }
  return r;
}
__global__ __launch_bounds__(EW_BLOCK) void scalar2_generic(int k, DevShape sz, DevShape sx, int zdt, int xdt, void* z, const void* x,
                                                            LongType n, double s1, double s2) {
  const LongType step = (LongType)gridDim.x * EW_BLOCK;
  for (LongType i = (LongType)blockIdx.x * EW_BLOCK + threadIdx.x; i < n; i += step) {
    const LongType oz = walk<LongType>(sz, i), ox = walk<LongType>(sx, i);
    store_any(z, zdt, oz, scalar2_eval(k, load_any(x, xdt, ox), xdt == DOUBLE, s1, s2));
  }
}
// the same on dense arrays of one float type: 16-byte vectors, one per thread, and a scalar tail
template <typename T>
__global__ __launch_bounds__(EW_BLOCK) void scalar2_contig(int k, const T* __restrict__ x, T* __restrict__ z, LongType n, double s1, double s2) {
  constexpr int V = 16 / sizeof(T);
  using IO = RawIO<T>;
  using RT = typename IO::raw;
  using A = typename Conv<T>::acc;
  constexpr bool DBL = sizeof(T) == 8;
  const LongType nvec = n / V;
  const LongType i = (LongType)blockIdx.x * EW_BLOCK + threadIdx.x;
  if (i < nvec) {
    A a[V];
    IO::unpack(*(reinterpret_cast<const RT*>(x) + i), a);
#pragma unroll
    for (int e = 0; e < V; e++) {
      const double r = scalar2_eval(k, (double)a[e], DBL, s1, s2);
      a[e] = DBL ? (A)r : (A)(float)r;
    }
    *(reinterpret_cast<RT*>(z) + i) = IO::pack(a);
  }
  const LongType tail = nvec * V + i;
  if (tail < n) {
    const double r = scalar2_eval(k, (double)to_float(x[tail]), DBL, s1, s2);
    z[tail] = Conv<T>::from(DBL ? (A)r : (A)(float)r);
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
// Which accesses of a dense streaming op are non-temporal, by the bytes it moves (measured cold, over rotating operand sets,
// on 50 MB - 270 MB transforms): 0 = none below 8 MiB; 2 = stores only up to the size of the last-level cache -- written
// with ordinary stores the output sits dirty in L2 until the kernel ends and is flushed then, which the next launch waits
// for (gelu bf16 [16,1024,768]: 10.8 -> 8.5 us per launch; a consumer that reads the result right away loses 3 % to it);
// 3 = loads and stores for what cannot stay in the cache anyway.
static int streamPolicy(size_t bytes) { return bytes > ((size_t)288 << 20) ? 3 : bytes >= ((size_t)8 << 20) ? 2 : 0; }
static bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

// A row vector against a dense [rows, cols] array whose row length is not a whole number of 16-byte vectors (or whose operands
// start off 16-byte boundaries), which keeps it off the vector path of ew_nd: the dense array as one run of element-aligned
// 16-byte vectors, one remainder per vector for the column of its first element, its stretch
// of the row vector another such load (element by element where the vector runs over the end of a row).  bf16 [16000, 770] + [770]: 23.9 us with one element per thread.
template <typename F, typename T>
__global__ __launch_bounds__(EW_BLOCK) void row_broadcast_flat(const T* __restrict__ x, const T* __restrict__ v, T* __restrict__ z, LongType n, LongType cols,
                                                               int nts) {
  constexpr int V = 16 / sizeof(T);
  using VT = Vec<T, V>;
  using A = typename Conv<T>::acc;
  const LongType nvec = n / V;
  const LongType step = (LongType)gridDim.x * EW_BLOCK;
  const bool small = n < ((LongType)1 << 32);
  for (LongType i = (LongType)blockIdx.x * EW_BLOCK + threadIdx.x; i < nvec; i += step) {
    VT a, out;
    __builtin_memcpy(&a, x + i * V, sizeof(VT));
    LongType c = small ? (LongType)((unsigned)(i * V) % (unsigned)cols) : (i * V) % cols;
    if (c + V <= cols) {   // the usual case: the vector lies inside one row, its stretch of the row vector is one load too
      VT b;
      __builtin_memcpy(&b, v + c, sizeof(VT));
#pragma unroll
      for (int e = 0; e < V; e++) out.v[e] = Conv<T>::from(F::template apply<A>((A)to_float(a.v[e]), (A)to_float(b.v[e])));
    } else {
#pragma unroll
      for (int e = 0; e < V; e++) {
        out.v[e] = Conv<T>::from(F::template apply<A>((A)to_float(a.v[e]), (A)to_float(v[c])));
        c = c + 1 == cols ? 0 : c + 1;
      }
    }
    if (nts) nt_store16_elem_aligned(z + i * V, out);
    else __builtin_memcpy(z + i * V, &out, sizeof(VT));
  }
  const LongType j = nvec * V + (LongType)blockIdx.x * EW_BLOCK + threadIdx.x;   // the up to V - 1 elements that are left
  if (j < n) z[j] = Conv<T>::from(F::template apply<A>((A)to_float(x[j]), (A)to_float(v[j % cols])));
}
template <typename F2, typename T, int NIN>
static void launchNd(hipStream_t s, const EwPlan& p, const T* x, const T* y, T* z) {
  constexpr int V = 16 / sizeof(T);
  NdArgs a;
  a.rank = p.rank;
  for (int d = 0; d < p.rank; d++) {
    a.shape[d] = p.shape[d];
    for (int o = 0; o < 3; o++) a.stride[o][d] = p.stride[o][d];
  }
  a.nts = streamPolicy(sizeof(T) * (size_t)p.length) >= 2 ? 1 : 0;
  const LongType inner = p.shape[p.rank - 1];
  // vectors along the inner axis: the output and every input run along it with unit stride from aligned starts -- or an
  // input repeats along it (stride 0), which needs no alignment
  bool vec = inner % V == 0 && aligned16(z);
  for (int o = 0; o <= NIN && vec; o++) {
    const LongType is = p.stride[o][p.rank - 1];
    if (o > 0 && is == 0) continue;
    if (is != 1 || !aligned16(o == 0 ? (const void*)z : o == 1 ? (const void*)x : (const void*)y)) vec = false;
    for (int d = 0; d < p.rank - 1; d++) if (p.stride[o][d] % V != 0) vec = false;
  }
  if (vec) {
    LongType cpr = inner / V, total = p.length / V;
    if (p.index32) hipLaunchKernelGGL((ew_nd<F2, T, NIN, V, unsigned>), dim3(gridFor(total, EW_BLOCK)), dim3(EW_BLOCK), 0, s, a, x, y, z, (unsigned)cpr, (unsigned)total);
    else hipLaunchKernelGGL((ew_nd<F2, T, NIN, V, unsigned long long>), dim3(gridFor(total, EW_BLOCK)), dim3(EW_BLOCK), 0, s, a, x, y, z, (unsigned long long)cpr, (unsigned long long)total);
  } else {
    if constexpr (NIN == 2 && sizeof(T) <= 4) {
      // x and z dense [rows, cols], y a row vector of cols elements
      if (p.rank == 2 && p.stride[0][1] == 1 && p.stride[0][0] == inner && p.stride[1][1] == 1 && p.stride[1][0] == inner && p.stride[2][1] == 1 &&
          p.stride[2][0] == 0 && p.length >= V && inner < ((LongType)1 << 31)) {
        hipLaunchKernelGGL((row_broadcast_flat<F2, T>), dim3(gridFor(p.length / V, EW_BLOCK)), dim3(EW_BLOCK), 0, s, x, y, z, p.length, inner, a.nts);
        return;
      }
    }
    LongType cpr = inner, total = p.length;
    if (p.index32) hipLaunchKernelGGL((ew_nd<F2, T, NIN, 1, unsigned>), dim3(gridFor(total, EW_BLOCK)), dim3(EW_BLOCK), 0, s, a, x, y, z, (unsigned)cpr, (unsigned)total);
    else hipLaunchKernelGGL((ew_nd<F2, T, NIN, 1, unsigned long long>), dim3(gridFor(total, EW_BLOCK)), dim3(EW_BLOCK), 0, s, a, x, y, z, (unsigned long long)cpr, (unsigned long long)total);
  }
}

// ---- copies that transpose: z runs along one axis, x along another ---------------------------------------------------------
// A 64 x 64 tile goes through LDS: read along x's contiguous axis (axis A), written along z's (the last axis), both sides in
// whole 64-element runs; the other axes are a batch walked per block.  Rows of 65 keep the transposed LDS reads conflict-free.
struct TransposeArgs {
  LongType nA, nB, xB, zA;          // extents of the two axes; x's stride along z's axis, z's stride along x's axis
  int nOther;
  LongType oShape[MAX_DEV_RANK], oX[MAX_DEV_RANK], oZ[MAX_DEV_RANK];
  unsigned tilesA, tilesB;
};
// NTS: the result leaves through non-temporal stores (the host asks for them from 8 MiB on, see streamPolicy)
template <typename T, bool NTS>
__global__ __launch_bounds__(256) void transpose_tiled(TransposeArgs a, const T* __restrict__ x, T* __restrict__ z) {
  __shared__ T tile[64][65];
  const unsigned tb = blockIdx.x % a.tilesB, ta = blockIdx.x / a.tilesB;
  LongType rest = blockIdx.y, xo = 0, zo = 0;
  for (int d = a.nOther - 1; d >= 0; d--) { const LongType q = rest / a.oShape[d], c = rest - q * a.oShape[d]; xo += c * a.oX[d]; zo += c * a.oZ[d]; rest = q; }
  const LongType a0 = (LongType)ta * 64, b0 = (LongType)tb * 64;
  if constexpr (sizeof(T) <= 4) {
    // whole tiles: 16 bytes per lane on both sides of the copy (element-aligned vectors: any row pitch, any start), the
    // transposition itself in LDS element by element -- with rows of 65 a wave's writes (4 or 8 tile rows, every V-th
    // column) and its transposed reads both fall on every bank equally often
    if (a0 + 64 <= a.nA && b0 + 64 <= a.nB) {
      constexpr int V = 16 / sizeof(T), CPR = 64 / V, PER = 64 * CPR / 256;   // vectors per tile row, per thread
      struct alignas(sizeof(T)) Pack { T e[V]; };
      const int c = threadIdx.x % CPR, r = threadIdx.x / CPR;
      Pack in[PER];
#pragma unroll
      for (int u = 0; u < PER; u++) {
        const int j = r + u * (256 / CPR);
        __builtin_memcpy(&in[u], x + xo + (a0 + c * V) + (b0 + j) * a.xB, sizeof(Pack));
      }
#pragma unroll
      for (int u = 0; u < PER; u++) {
        const int j = r + u * (256 / CPR);
#pragma unroll
        for (int e = 0; e < V; e++) tile[j][c * V + e] = in[u].e[e];
      }
      __syncthreads();
#pragma unroll
      for (int u = 0; u < PER; u++) {
        const int i = r + u * (256 / CPR);
        Pack out;
#pragma unroll
        for (int e = 0; e < V; e++) out.e[e] = tile[c * V + e][i];
        T* dst = z + zo + (a0 + i) * a.zA + (b0 + c * V);
        if constexpr (NTS) {
          nt_store16_elem_aligned(dst, out);
        } else {
          __builtin_memcpy(dst, &out, sizeof(Pack));
        }
      }
      return;
    }
  }
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  if (a0 + tx < a.nA) {
#pragma unroll 4
    for (int j = ty; j < 64; j += 4)
      if (b0 + j < a.nB) tile[j][tx] = x[xo + (a0 + tx) + (b0 + j) * a.xB];
  }
  __syncthreads();
  if (b0 + tx < a.nB) {
#pragma unroll 4
    for (int j = ty; j < 64; j += 4)
      if (a0 + j < a.nA) z[zo + (a0 + j) * a.zA + (b0 + tx)] = tile[tx][j];
  }
}
// whether the copy described by p (operand 0: z, operand 1: x) is such a transpose; launches it if so
template <typename T>
static bool tryTransposeCopy(hipStream_t s, const EwPlan& p, const T* x, T* z) {
  const int r = p.rank;
  if (r < 2 || p.stride[0][r - 1] != 1 || p.stride[1][r - 1] == 1) return false;
  int dA = -1;
  for (int d = 0; d < r - 1; d++) if (p.stride[1][d] == 1 && p.shape[d] > 1) dA = d;
  if (dA < 0 || p.shape[dA] < 16 || p.shape[r - 1] < 16) return false;
  TransposeArgs a;
  a.nA = p.shape[dA]; a.nB = p.shape[r - 1]; a.xB = p.stride[1][r - 1]; a.zA = p.stride[0][dA];
  a.nOther = 0;
  LongType batch = 1;
  for (int d = 0; d < r - 1; d++) {
    if (d == dA) continue;
    a.oShape[a.nOther] = p.shape[d]; a.oX[a.nOther] = p.stride[1][d]; a.oZ[a.nOther] = p.stride[0][d]; a.nOther++;
    batch *= p.shape[d];
  }
  a.tilesA = (unsigned)((a.nA + 63) / 64); a.tilesB = (unsigned)((a.nB + 63) / 64);
  if (batch > 65535 || (LongType)a.tilesA * a.tilesB >= (1LL << 31)) return false;
  if (streamPolicy(sizeof(T) * (size_t)p.length) >= 2) hipLaunchKernelGGL((transpose_tiled<T, true>), dim3(a.tilesA * a.tilesB, (unsigned)batch), dim3(256), 0, s, a, x, z);
  else hipLaunchKernelGGL((transpose_tiled<T, false>), dim3(a.tilesA * a.tilesB, (unsigned)batch), dim3(256), 0, s, a, x, z);
  return true;
}

template <int K, typename T>
static void unaryTyped(hipStream_t s, const EwPlan& p, const void* x, void* z) {
  const T* xt = (const T*)x;
  T* zt = (T*)z;
  if (p.contiguous && aligned16(x) && aligned16(z)) {
    constexpr int V = 16 / sizeof(T);
    const unsigned grid = (unsigned)((p.length / V + EW_BLOCK) / EW_BLOCK);
    const int nt = streamPolicy(2 * sizeof(T) * (size_t)p.length);
    if (nt == 3) hipLaunchKernelGGL((unary_contig<Unary<K>, T, true, true>), dim3(grid), dim3(EW_BLOCK), 0, s, xt, zt, p.length);
    else if (nt == 2) hipLaunchKernelGGL((unary_contig<Unary<K>, T, false, true>), dim3(grid), dim3(EW_BLOCK), 0, s, xt, zt, p.length);
    else hipLaunchKernelGGL((unary_contig<Unary<K>, T, false, false>), dim3(grid), dim3(EW_BLOCK), 0, s, xt, zt, p.length);
  } else {
    if (K == U_IDENTITY && x != z && tryTransposeCopy<T>(s, p, xt, zt)) return;
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

template <typename T, int NIN>
static void tailContigTyped(hipStream_t s, int k, const void* x, const void* y, void* z, LongType n) {
  constexpr int V = 16 / sizeof(T);
  const unsigned grid = (unsigned)((n / V + EW_BLOCK) / EW_BLOCK);
  hipLaunchKernelGGL((tail_contig<T, NIN>), dim3(grid), dim3(EW_BLOCK), 0, s, k, (const T*)x, (const T*)y, (T*)z, n);
}
template <int NIN>
static bool tailContig(hipStream_t s, int k, DataType dt, const void* x, const void* y, void* z, LongType n) {
  switch (dt) {
    case FLOAT32: tailContigTyped<float, NIN>(s, k, x, y, z, n); return true;
    case DOUBLE: tailContigTyped<double, NIN>(s, k, x, y, z, n); return true;
    case HALF: tailContigTyped<f16_t, NIN>(s, k, x, y, z, n); return true;
    case BFLOAT16: tailContigTyped<bf16_t, NIN>(s, k, x, y, z, n); return true;
    default: return false;
  }
}

// ---- dense casts between fp32 and the 16-bit types (the assign loop between two types) -------------------------------------
// eight elements per thread: the wider side moves as two 16-byte vectors, the narrower as one; the tail one by one
template <typename TI, typename TO, bool NTS>
__global__ __launch_bounds__(EW_BLOCK) void cast_contig(const TI* __restrict__ x, TO* __restrict__ z, LongType n) {
  const LongType i = ((LongType)blockIdx.x * EW_BLOCK + threadIdx.x) * 8;
  if (i + 8 <= n) {
    Vec<TI, 8> v = *reinterpret_cast<const Vec<TI, 8>*>(x + i);
    Vec<TO, 8> o;
#pragma unroll
    for (int e = 0; e < 8; e++) o.v[e] = Conv<TO>::from(to_float(v.v[e]));
    if constexpr (NTS) {
      struct Quads { raw_u32x4 q[sizeof(TO) * 8 / 16]; };
      const Quads qs = __builtin_bit_cast(Quads, o);
#pragma unroll
      for (int k = 0; k < (int)(sizeof(TO) * 8 / 16); k++) __builtin_nontemporal_store(qs.q[k], reinterpret_cast<raw_u32x4*>(z + i) + k);
    } else {
      *reinterpret_cast<Vec<TO, 8>*>(z + i) = o;
    }
  } else {
    for (LongType j = i; j < n; j++) z[j] = Conv<TO>::from(to_float(x[j]));
  }
}
template <typename TI>
static bool castFrom(hipStream_t s, DataType zdt, const void* x, void* z, LongType n) {
  const unsigned grid = (unsigned)((n / 8 + EW_BLOCK) / EW_BLOCK);
#define ND4J_CAST(TO) do { if (streamPolicy(sizeof(TO) * (size_t)n) >= 2) hipLaunchKernelGGL((cast_contig<TI, TO, true>), dim3(grid), dim3(EW_BLOCK), 0, s, (const TI*)x, (TO*)z, n); \
                           else hipLaunchKernelGGL((cast_contig<TI, TO, false>), dim3(grid), dim3(EW_BLOCK), 0, s, (const TI*)x, (TO*)z, n); } while (0)
  switch (zdt) {
    case FLOAT32: if constexpr (!std::is_same<TI, float>::value) { ND4J_CAST(float); return true; } break;
    case HALF: if constexpr (!std::is_same<TI, f16_t>::value) { ND4J_CAST(f16_t); return true; } break;
    case BFLOAT16: if constexpr (!std::is_same<TI, bf16_t>::value) { ND4J_CAST(bf16_t); return true; } break;
    default: break;
  }
#undef ND4J_CAST
  return false;
}
static bool tryCastContig(hipStream_t s, DataType xdt, DataType zdt, const void* x, void* z, const EwPlan& p) {
  if (xdt == zdt || !p.sameShape || !p.contiguous || ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(z)) & 31) != 0 || p.length >= (1LL << 40)) return false;
  switch (xdt) {
    case FLOAT32: return castFrom<float>(s, zdt, x, z, p.length);
    case HALF: return castFrom<f16_t>(s, zdt, x, z, p.length);
    case BFLOAT16: return castFrom<bf16_t>(s, zdt, x, z, p.length);
    default: return false;
  }
}

void launchUnary(hipStream_t s, UnaryKind k, DataType xdt, DataType zdt, const void* x, void* z, const EwPlan& p) {
  if (p.length == 0) return;
  if (k == U_IDENTITY && tryCastContig(s, xdt, zdt, x, z, p)) { HIP_CHECK(hipGetLastError()); return; }
  if (isIntLike(xdt) && isIntLike(zdt)) return launchIntElementwise(s, k, false, xdt, xdt, zdt, x, nullptr, z, p, 0, false);
  if (k >= U_TAIL_FIRST && k < U_TAIL_END) {
    if (!(p.sameShape && xdt == zdt && p.contiguous && aligned16(x) && aligned16(z) && tailContig<1>(s, k, xdt, x, x, z, p.length)))
      hipLaunchKernelGGL((tail_generic<1>), dim3(gridFor(p.length, EW_BLOCK)), dim3(EW_BLOCK), 0, s, (int)k, p.own[0], p.own[1], p.own[1],
                         (int)zdt, (int)xdt, (int)xdt, z, x, x, p.length, 0.0, 0);
    HIP_CHECK(hipGetLastError());
    return;
  }
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
    const int nt = streamPolicy(3 * sizeof(T) * (size_t)p.length);
    if (nt == 3) hipLaunchKernelGGL((pairwise_contig<Pairwise<K>, T, true, true>), dim3(grid), dim3(EW_BLOCK), 0, s, xt, yt, zt, p.length);
    else if (nt == 2) hipLaunchKernelGGL((pairwise_contig<Pairwise<K>, T, false, true>), dim3(grid), dim3(EW_BLOCK), 0, s, xt, yt, zt, p.length);
    else hipLaunchKernelGGL((pairwise_contig<Pairwise<K>, T, false, false>), dim3(grid), dim3(EW_BLOCK), 0, s, xt, yt, zt, p.length);
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
  if (isIntLike(xdt) && isIntLike(ydt) && isIntLike(zdt)) return launchIntElementwise(s, k, true, xdt, ydt, zdt, x, y, z, p, 0, false);
  if (k >= P_TAIL_FIRST && k < P_TAIL_END) {
    if (!(p.sameShape && xdt == zdt && ydt == zdt && p.contiguous && aligned16(x) && aligned16(y) && aligned16(z) &&
          tailContig<2>(s, k, zdt, x, y, z, p.length)))
      hipLaunchKernelGGL((tail_generic<2>), dim3(gridFor(p.length, EW_BLOCK)), dim3(EW_BLOCK), 0, s, (int)k, p.own[0], p.own[1], p.own[2],
                         (int)zdt, (int)xdt, (int)ydt, z, x, y, p.length, 0.0, 0);
    HIP_CHECK(hipGetLastError());
    return;
  }
  switch (k) {
#define CASE(K) case K: pairwiseKind<K>(s, xdt, ydt, zdt, x, y, z, p); break;
    CASE(P_ADD) CASE(P_COPY) CASE(P_DIV) CASE(P_MUL) CASE(P_RSUB) CASE(P_SUB) CASE(P_MAX) CASE(P_MIN) CASE(P_RDIV)
    CASE(P_SQSUB)
#undef CASE
    default: ND4J_THROW("launchPairwise: unknown op kind");
  }
  HIP_CHECK(hipGetLastError());
}

// ---- scalar ops ----------------------------------------------------------------------------------------------

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
// 16 bytes per thread along unit-stride inner runs; a dense array is one run whose last few elements go one by one
template <typename F, typename T, typename I>
__global__ __launch_bounds__(EW_BLOCK) void scalar_nd_vec(NdArgs a, const T* __restrict__ x, T* __restrict__ z,
                                                          typename Conv<T>::acc sc, I chunksPerRow, I totalChunks, LongType n) {
  using A = typename Conv<T>::acc;
  constexpr int V = 16 / sizeof(T);
  using VT = Vec<T, V>;
  const I step = (I)gridDim.x * EW_BLOCK;
  for (I c = (I)blockIdx.x * EW_BLOCK + threadIdx.x; c < totalChunks; c += step) {
    LongType oz, ox;
    if (a.rank == 1) {   // a dense array: one run, no division
      oz = ox = (LongType)c * V;
    } else {
      I outer = c / chunksPerRow;
      const LongType inner = (LongType)(c - outer * chunksPerRow) * V;
      oz = inner; ox = inner;
#pragma unroll 1
      for (int d = a.rank - 2; d >= 0; d--) {
        const I dim = (I)a.shape[d];
        const I q = outer / dim;
        const LongType cd = (LongType)(outer - q * dim);
        oz += cd * a.stride[0][d]; ox += cd * a.stride[1][d];
        outer = q;
      }
    }
    const VT vx = *reinterpret_cast<const VT*>(x + ox);
    VT out;
#pragma unroll
    for (int e = 0; e < V; e++) out.v[e] = Conv<T>::from(F::template apply<A>((A)to_float(vx.v[e]), sc));
    store_vec(reinterpret_cast<VT*>(z + oz), out, a.nts != 0);
  }
  // rank 1 only: what is left after the last whole vector
  if (blockIdx.x == 0) {
    const LongType i = (LongType)totalChunks * V + threadIdx.x;
    if (a.rank == 1 && i < n) z[i] = Conv<T>::from(F::template apply<A>((A)to_float(x[i]), sc));
  }
}
template <int K, typename T>
static void scalarTyped(hipStream_t s, const void* x, double sc, void* z, const EwPlan& p) {
  NdArgs a;
  a.rank = p.rank;
  for (int d = 0; d < p.rank; d++) { a.shape[d] = p.shape[d]; for (int o = 0; o < 3; o++) a.stride[o][d] = p.stride[o][d]; }
  a.nts = streamPolicy(sizeof(T) * (size_t)p.length) >= 2 ? 1 : 0;
  using A = typename Conv<T>::acc;
  A scv = (A)sc;
  constexpr int V = 16 / sizeof(T);
  const LongType inner = p.shape[p.rank - 1];
  bool vec = aligned16(x) && aligned16(z) && p.stride[0][p.rank - 1] == 1 && p.stride[1][p.rank - 1] == 1 &&
             (p.rank == 1 ? inner >= V : inner % V == 0);
  for (int d = 0; d < p.rank - 1 && vec; d++) if (p.stride[0][d] % V != 0 || p.stride[1][d] % V != 0) vec = false;
  if (vec) {
    const LongType cpr = inner / V, total = p.rank == 1 ? cpr : p.length / V;
    if (p.index32) hipLaunchKernelGGL((scalar_nd_vec<Pairwise<K>, T, unsigned>), dim3(gridFor(total, EW_BLOCK)), dim3(EW_BLOCK), 0, s, a, (const T*)x, (T*)z, scv, (unsigned)cpr, (unsigned)total, p.length);
    else hipLaunchKernelGGL((scalar_nd_vec<Pairwise<K>, T, unsigned long long>), dim3(gridFor(total, EW_BLOCK)), dim3(EW_BLOCK), 0, s, a, (const T*)x, (T*)z, scv, (unsigned long long)cpr, (unsigned long long)total, p.length);
    return;
  }
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
  if (isIntLike(dt)) return launchIntElementwise(s, k, true, dt, dt, dt, x, nullptr, z, p, (LongType)scalar, true);
  if (k >= P_TAIL_FIRST && k < P_TAIL_END) {
    // the scalar takes the array's storage type first, as the reference holds it in an array of that type
    hipLaunchKernelGGL((tail_generic<2>), dim3(gridFor(p.length, EW_BLOCK)), dim3(EW_BLOCK), 0, s, (int)k,
                       p.own[0], p.own[1], p.own[1], (int)dt, (int)dt, (int)dt, z, x, x, p.length, scalar, 1);
    HIP_CHECK(hipGetLastError());
    return;
  }
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

void launchScalar2Op(hipStream_t s, Scalar2Kind k, DataType xdt, DataType zdt, const void* x, double s1, double s2, void* z,
                     const EwPlan& p) {
  if (p.length == 0) return;
  if (p.sameShape && p.contiguous && xdt == zdt && ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(z)) & 15) == 0 &&
      (xdt == FLOAT32 || xdt == DOUBLE || xdt == HALF || xdt == BFLOAT16)) {
    const LongType V = 16 / (LongType)sizeOf(xdt);
    const dim3 grid((unsigned)((p.length / V + EW_BLOCK) / EW_BLOCK));   // one vector per thread; the block after the last whole one holds the tail
    switch (xdt) {
      case FLOAT32: hipLaunchKernelGGL((scalar2_contig<float>), grid, dim3(EW_BLOCK), 0, s, (int)k, (const float*)x, (float*)z, p.length, s1, s2); break;
      case DOUBLE: hipLaunchKernelGGL((scalar2_contig<double>), grid, dim3(EW_BLOCK), 0, s, (int)k, (const double*)x, (double*)z, p.length, s1, s2); break;
      case HALF: hipLaunchKernelGGL((scalar2_contig<f16_t>), grid, dim3(EW_BLOCK), 0, s, (int)k, (const f16_t*)x, (f16_t*)z, p.length, s1, s2); break;
      default: hipLaunchKernelGGL((scalar2_contig<bf16_t>), grid, dim3(EW_BLOCK), 0, s, (int)k, (const bf16_t*)x, (bf16_t*)z, p.length, s1, s2); break;
    }
    HIP_CHECK(hipGetLastError());
    return;
  }
  hipLaunchKernelGGL(scalar2_generic, dim3(gridFor(p.length, EW_BLOCK)), dim3(EW_BLOCK), 0, s, (int)k, p.own[0], p.own[1], (int)zdt,
                     (int)xdt, z, x, p.length, s1, s2);
  HIP_CHECK(hipGetLastError());
}

// ---- gather rows / fill ------------------------------------------------------------------------------------
template <typename T, typename IT>
__global__ __launch_bounds__(EW_BLOCK) void gather_rows(const T* __restrict__ table, const IT* __restrict__ idx,
                                                        T* __restrict__ z, LongType nIdx, LongType rowLen, LongType tableRows, int nts) {
  const LongType n = nIdx * rowLen;
  const LongType step = (LongType)gridDim.x * EW_BLOCK;
  for (LongType i = (LongType)blockIdx.x * EW_BLOCK + threadIdx.x; i < n; i += step) {
    LongType r = i / rowLen, c = i - r * rowLen;
    LongType src = (LongType)idx[r];
    if (src < 0) src += tableRows;
    // out-of-range ids are clamped so that a bad id cannot fault the device; the host validates ids it can see
    src = src < 0 ? 0 : (src >= tableRows ? tableRows - 1 : src);
    store_vec(z + i, table[src * rowLen + c], nts != 0);
  }
}
void launchGatherRows(hipStream_t s, DataType dt, DataType idxDt, const void* table, const void* idx, void* z,
                      LongType nIdx, LongType rowLen, LongType tableRows) {
  if (nIdx * rowLen == 0) return;
  ND4J_REQUIRE(idxDt == INT32 || idxDt == INT64, "gather: indices must be INT32 or INT64");
  dim3 g(gridFor(nIdx * rowLen, EW_BLOCK)), b(EW_BLOCK);
  const int nts = streamPolicy((size_t)(nIdx * rowLen) * sizeOf(dt)) >= 2 ? 1 : 0;   // only the 16-byte rows take it
#define GATHER(T)                                                                                                         \
  if (idxDt == INT32) hipLaunchKernelGGL((gather_rows<T, int>), g, b, 0, s, (const T*)table, (const int*)idx, (T*)z, nIdx, rowLen, tableRows, nts); \
  else hipLaunchKernelGGL((gather_rows<T, LongType>), g, b, 0, s, (const T*)table, (const LongType*)idx, (T*)z, nIdx, rowLen, tableRows, nts);
  // rows that are whole 16-byte units in aligned arrays move as such
  using U16 = Vec<unsigned, 4>;
  const LongType es = (LongType)sizeOf(dt);
  if ((rowLen * es) % 16 == 0 && aligned16(table) && aligned16(z)) {
    const LongType units = rowLen * es / 16;
    g = dim3(gridFor(nIdx * units, EW_BLOCK));
    rowLen = units;
    GATHER(U16)
    HIP_CHECK(hipGetLastError());
    return;
  }
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
