/*
 * CPU oracle for the libnd4j data-parallel op path -- TEST INFRASTRUCTURE ONLY.
 * See nd4j_oracle.h for conventions and for what pins each function.
 * All reference paths below are relative to libnd4j/include/ of the reference tree.
 */
#define _GNU_SOURCE
#include "nd4j_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define ORC_MAX_RANK 32

/* ---------------------------------------------------------------------------------------------
 * shapeInfo descriptor                      helpers/shape.h:76-104 (extra index), :1804-1822
 * ------------------------------------------------------------------------------------------- */
static inline int si_rank(const int64_t *si) { return (int)si[0]; }
static inline const int64_t *si_shape(const int64_t *si) { return si + 1; }
static inline const int64_t *si_stride(const int64_t *si) { return si + 1 + si_rank(si); }
/* rank 0 keeps the flags word at index 3 (descriptor length 6); otherwise at 2*rank+1 */
static inline int64_t si_extra(const int64_t *si) { return si_rank(si) == 0 ? si[3] : si[2 * si_rank(si) + 1]; }

int64_t orc_shape_info_length(int rank) { return rank == 0 ? 6 : 2 * (int64_t)rank + 4; }

/* dtype bits of the flags word               array/ArrayOptions.h:41-97, ArrayOptions.hXX:198-276 */
static int64_t dtype_flag(int dtype) {
  switch (dtype) {
    case ORC_HALF: return 4096;
    case ORC_BFLOAT16: return 2048;
    case ORC_FLOAT32: return 8192;
    case ORC_DOUBLE: return 16384;
    case ORC_INT32: return 131072;
    case ORC_INT64: return 262144;
    case ORC_BOOL: return 524288;
    default: return 0;
  }
}

int orc_dtype(const int64_t *si) {
  int64_t e = si_extra(si);
  if (e & 8388608) return 255; /* unsigned flavours are not on this path */
  if (e & 8192) return ORC_FLOAT32;
  if (e & 16384) return ORC_DOUBLE;
  if (e & 4096) return ORC_HALF;
  if (e & 2048) return ORC_BFLOAT16;
  if (e & 524288) return ORC_BOOL;
  if (e & 131072) return ORC_INT32;
  if (e & 262144) return ORC_INT64;
  return 255;
}

void orc_make_shape_info(int rank, const int64_t *shape, const int64_t *strides, int dtype, char order, int64_t *out) {
  if (rank == 0) {
    out[0] = 0; out[1] = 0; out[2] = 1; out[3] = dtype_flag(dtype); out[4] = 1; out[5] = order;
    return;
  }
  out[0] = rank;
  for (int i = 0; i < rank; i++) out[1 + i] = shape[i];
  if (strides) {
    for (int i = 0; i < rank; i++) out[1 + rank + i] = strides[i];
  } else if (order == 'c') {
    int64_t s = 1;
    for (int i = rank - 1; i >= 0; i--) { out[1 + rank + i] = s; s *= shape[i]; }
  } else {
    int64_t s = 1;
    for (int i = 0; i < rank; i++) { out[1 + rank + i] = s; s *= shape[i]; }
  }
  out[2 * rank + 1] = dtype_flag(dtype);
  out[2 * rank + 2] = strides ? 0 : 1;
  out[2 * rank + 3] = order;
}

int64_t orc_length(const int64_t *si) {
  int r = si_rank(si);
  if (si_extra(si) & 8) return 0; /* ARRAY_EMPTY */
  int64_t n = 1;
  for (int i = 0; i < r; i++) n *= si_shape(si)[i];
  return n;
}

/* INDEX2COORDS walks the SHAPE row-major whatever the order flag says, then COORDS2INDEX takes
 * the dot product with the strides.           helpers/shape.h:588-676, :678-740 */
int64_t orc_offset(const int64_t *si, int64_t idx) {
  int r = si_rank(si);
  const int64_t *sh = si_shape(si), *st = si_stride(si);
  int64_t off = 0;
  for (int i = r - 1; i > 0; i--) {
    off += (idx % sh[i]) * st[i];
    idx /= sh[i];
  }
  if (r > 0) off += idx * st[0];
  return off;
}

/* ---------------------------------------------------------------------------------------------
 * half types                                 types/bfloat16.h:186-213 (RNE, NaN -> 0x7FC0)
 * ------------------------------------------------------------------------------------------- */
uint16_t orc_f32_to_bf16(float f) {
  if (isnan(f)) return 0x7FC0;
  union { float f; uint32_t i; } u;
  u.f = f;
  uint32_t lsb = (u.i >> 16) & 1;
  u.i += 0x7fff + lsb;
  return (uint16_t)(u.i >> 16);
}
float orc_bf16_to_f32(uint16_t h) {
  union { float f; uint32_t i; } u;
  u.i = ((uint32_t)h) << 16;
  return u.f;
}
/* IEEE binary16, round-to-nearest-even (what cpu_float2ihalf_rn produces, types/float16.h:338-349) */
uint16_t orc_f32_to_f16(float f) {
  union { float f; uint32_t i; } u;
  u.f = f;
  uint32_t x = u.i;
  uint16_t sign = (uint16_t)((x >> 16) & 0x8000);
  uint32_t ax = x & 0x7fffffff;
  if (ax >= 0x7f800000) return (uint16_t)(sign | (ax > 0x7f800000 ? 0x7e00 : 0x7c00));
  if (ax >= 0x477ff000) return (uint16_t)(sign | 0x7c00); /* rounds to inf */
  if (ax < 0x33000001) return sign;                       /* rounds to zero */
  int32_t e = (int32_t)(ax >> 23) - 127;
  uint32_t m = (ax & 0x7fffff) | 0x800000;
  if (e < -14) { /* subnormal half */
    int shift = -e - 14 + 13;
    uint32_t v = m >> shift;
    uint32_t rem = m & ((1u << shift) - 1), halfway = 1u << (shift - 1);
    if (rem > halfway || (rem == halfway && (v & 1))) v++;
    return (uint16_t)(sign | v);
  }
  uint32_t v = ((uint32_t)(e + 15) << 10) | ((m >> 13) & 0x3ff);
  uint32_t rem = m & 0x1fff;
  if (rem > 0x1000 || (rem == 0x1000 && (v & 1))) v++;
  return (uint16_t)(sign | v);
}
float orc_f16_to_f32(uint16_t h) {
  uint32_t sign = ((uint32_t)h & 0x8000) << 16;
  uint32_t e = (h >> 10) & 0x1f, m = h & 0x3ff;
  union { float f; uint32_t i; } u;
  if (e == 0) {
    if (m == 0) { u.i = sign; return u.f; }
    float v = ldexpf((float)m, -24);
    return sign ? -v : v;
  }
  if (e == 31) { u.i = sign | 0x7f800000 | (m << 13); return u.f; }
  u.i = sign | ((e + 112) << 23) | (m << 13);
  return u.f;
}

static inline int dt_size(int dt) {
  switch (dt) {
    case ORC_HALF: case ORC_BFLOAT16: return 2;
    case ORC_FLOAT32: case ORC_INT32: return 4;
    case ORC_DOUBLE: case ORC_INT64: return 8;
    case ORC_BOOL: return 1;
    default: return 0;
  }
}
static inline int dt_is_float(int dt) { return dt == ORC_HALF || dt == ORC_BFLOAT16 || dt == ORC_FLOAT32 || dt == ORC_DOUBLE; }

static inline double ld(const void *p, int dt, int64_t off) {
  switch (dt) {
    case ORC_FLOAT32: return ((const float *)p)[off];
    case ORC_DOUBLE: return ((const double *)p)[off];
    case ORC_HALF: return orc_f16_to_f32(((const uint16_t *)p)[off]);
    case ORC_BFLOAT16: return orc_bf16_to_f32(((const uint16_t *)p)[off]);
    case ORC_INT32: return ((const int32_t *)p)[off];
    case ORC_INT64: return (double)((const int64_t *)p)[off];
    case ORC_BOOL: return ((const uint8_t *)p)[off];
    default: return NAN;
  }
}
static inline float ldf(const void *p, int dt, int64_t off) { return (float)ld(p, dt, off); }
static inline void st(void *p, int dt, int64_t off, double v) {
  switch (dt) {
    case ORC_FLOAT32: ((float *)p)[off] = (float)v; break;
    case ORC_DOUBLE: ((double *)p)[off] = v; break;
    case ORC_HALF: ((uint16_t *)p)[off] = orc_f32_to_f16((float)v); break;
    case ORC_BFLOAT16: ((uint16_t *)p)[off] = orc_f32_to_bf16((float)v); break;
    case ORC_INT32: ((int32_t *)p)[off] = (int32_t)v; break;
    case ORC_INT64: ((int64_t *)p)[off] = (int64_t)v; break;
    case ORC_BOOL: ((uint8_t *)p)[off] = v != 0; break;
    default: break;
  }
}
/* round a float through the storage type (what assigning to a T variable does in the reference) */
static inline float rnd(float v, int dt) {
  if (dt == ORC_HALF) return orc_f16_to_f32(orc_f32_to_f16(v));
  if (dt == ORC_BFLOAT16) return orc_bf16_to_f32(orc_f32_to_bf16(v));
  return v;
}

static int g_threads = 0;
void orc_set_threads(int n) { g_threads = n; }
int orc_get_threads(void) {
#ifdef _OPENMP
  return g_threads > 0 ? g_threads : omp_get_max_threads();
#else
  return 1;
#endif
}
#ifdef _OPENMP
#define PAR_FOR _Pragma("omp parallel for schedule(static) num_threads(orc_get_threads())")
#else
#define PAR_FOR
#endif

/* ---------------------------------------------------------------------------------------------
 * op-name hash                               helpers/impl/helper_hash.cpp:33-70, helper_hash.h:38-39
 * ------------------------------------------------------------------------------------------- */
int64_t orc_hash(const char *name) {
  static uint64_t table[256];
  static int init = 0;
  if (!init) {
    uint64_t h = 0x544B2FBACAAF1684ULL;
    for (int i = 0; i < 256; i++) {
      for (int j = 0; j < 31; j++) {
        h = (h >> 7) ^ h;
        h = (h << 11) ^ h;
        h = (h >> 10) ^ h;
      }
      table[i] = h;
    }
    init = 1;
  }
  uint64_t h = 0xBB40E64DA205B064ULL, mult = 7664345821815920749ULL;
  for (const char *c = name; *c; c++) {
    unsigned char uch = (unsigned char)*c;
    h = (h * mult) ^ table[uch & 0xff];
    h = (h * mult) ^ table[(uch >> 8) & 0xff]; /* always table[0]: the reference shifts an 8-bit value by 8 */
  }
  return (int64_t)h;
}

/* ---------------------------------------------------------------------------------------------
 * TAD pack                                   helpers/cpu/TadCalculator.cpp:25-100
 * sub-array keeps `dims` (ascending); offsets enumerate the remaining dims row-major.
 * ------------------------------------------------------------------------------------------- */
int64_t orc_tad(const int64_t *si, const int64_t *dims, int ndims, int64_t *tadSi, int64_t *offsets) {
  int r = si_rank(si);
  int keep[ORC_MAX_RANK] = {0};
  for (int i = 0; i < ndims; i++) {
    int64_t d = dims[i] < 0 ? dims[i] + r : dims[i];
    if (d < 0 || d >= r) return -1;
    keep[d] = 1;
  }
  int nk = 0;
  for (int i = 0; i < r; i++) nk += keep[i];
  int dt = orc_dtype(si);
  if (nk == 0 || nk == r) {
    /* all or nothing: the reference hands out scalar TADs with offsets 0..len-1 (TadCalculator.cpp:46-63) */
    int64_t n = orc_length(si);
    if (tadSi) orc_make_shape_info(0, NULL, NULL, dt, 'c', tadSi);
    if (offsets) for (int64_t i = 0; i < n; i++) offsets[i] = i;
    return n;
  }
  int64_t tshape[ORC_MAX_RANK], tstride[ORC_MAX_RANK], oshape[ORC_MAX_RANK], ostride[ORC_MAX_RANK];
  int tr = 0, orank = 0;
  for (int i = 0; i < r; i++) {
    if (keep[i]) { tshape[tr] = si_shape(si)[i]; tstride[tr++] = si_stride(si)[i]; }
    else { oshape[orank] = si_shape(si)[i]; ostride[orank++] = si_stride(si)[i]; }
  }
  if (tadSi) {
    orc_make_shape_info(tr, tshape, tstride, dt, (char)si[2 * r + 3], tadSi);
  }
  int64_t n = 1;
  for (int i = 0; i < orank; i++) n *= oshape[i];
  if (offsets) {
    for (int64_t t = 0; t < n; t++) {
      int64_t idx = t, off = 0;
      for (int i = orank - 1; i >= 0; i--) { off += (idx % oshape[i]) * ostride[i]; idx /= oshape[i]; }
      offsets[t] = off;
    }
  }
  return n;
}

/* ---------------------------------------------------------------------------------------------
 * scalar math                                math/templatemath.h
 * ------------------------------------------------------------------------------------------- */
/* sd_tanh<float>: copysign(1,x) * (1-p)/(1+p), p = powf((float)M_E, -2*|x|)   templatemath.h:1206-1223 */
static inline float ref_tanhf(float x) {
  float sign = copysignf(1.0f, x);
  float e = (float)M_E;
  float av = sign * x;
  float p = powf(e, -av * 2.f);
  return sign * ((1 - p) / (1 + p));
}
/* generic sd_tanh<T>: neg_tanh / pos_tanh   templatemath.h:1183-1204,1226-1230 */
static inline double ref_tanhd(double x) {
  double e = M_E;
  if (x <= 0) { double p = pow(e, x * 2.0); return (p - 1.0) / (p + 1.0); }
  double p = pow(e, x * -2.0);
  return (1.0 - p) / (1.0 + p);
}
static inline float ref_sigmoidf(float x) { return 1.0f / (1.0f + expf(-x)); }   /* templatemath.h:225-229 */
static inline double ref_sigmoidd(double x) { return 1.0 / (1.0 + exp(-x)); }

/* The rest of the TransformStrict table (loops/legacy_ops.h:54-64), restated from ops/ops.h and
 * math/templatemath.h (lines beside each case).  One body, expanded for float (libm *f functions, as the
 * reference's float path uses) and for double.  Not restated: 2 ScaledTanh, 3 Affine, 19 Stabilize, 25 SetRange
 * (extra parameters).  5 HardTanhDerivative and 10 HardSigmoidDerivative are declared through DECLARE_UNARY_CONDITIONAL_OP
 * (ops/op_macros_unary.h:109-113: (CONDITION) ? (TRUE_VAL) : (FALSE_VAL)) with the derivative's expression as the
 * CONDITION and d1 as both values (ops.h:222-226), so both return their input; 20 StabilizeFP16 (ops.h:381-384) returns
 * float16's smallest normal number, 2^-14 (DataTypeUtils::min<float16>, array/DataTypeUtils.h:463-465), for x <= 0. */
#define SELU_A 1.6732632423543772848170429916717
#define SELU_L 1.0507009873554804934193349852946
#define STRICT_TAIL(T, M, TANH, SIGM)                                                                         \
  switch (op) {                                                                                               \
    case 5: case 10: *out = x; return 0;                                      /* ops.h:222-226 */            \
    case 20: *out = x <= (T)0 ? (T)6.103515625e-05 : x; return 0;             /* ops.h:381-384 */            \
    case 4: { T t = TANH(x); *out = (T)1 - t * t; return 0; }                 /* templatemath.h:335-339 */   \
    case 6: { T g = SIGM(x); *out = g * ((T)1 - g); return 0; }               /* templatemath.h:343-347 */   \
    case 7: { T y = (T)1 + M(fabs)(x); *out = (T)1 / (y * y); return 0; }     /* templatemath.h:351-355 */   \
    case 8: *out = (T)1 / M(pow)(M(cos)(x), (T)2); return 0;                  /* ops.h:169 */                \
    case 9: *out = x > (T)0 ? (T)SELU_L : (T)SELU_A * (T)SELU_L * M(exp)(x); return 0;  /* ops.h:966-970 */  \
    case 11: {                                                                /* ops.h:1076-1086 */          \
      T dis = ((T)2 / (T)3) * x;                                                                              \
      T a = (T)1 + M(fabs)(dis) + M(pow)(dis, (T)2) + (T)1.41645f * M(pow)(dis, (T)4);                        \
      T sg = dis < 0 ? (T)-1 : dis > 0 ? (T)1 : (T)0;                                                         \
      T td = ((T)1 + sg * ((T)2 * dis + (T)4 * (T)1.41645f * M(pow)(dis, (T)3))) / (a * a);                   \
      *out = (T)1.7159f * ((T)2 / (T)3) * td; return 0;                                                       \
    }                                                                                                         \
    case 12: { if (x > (T)0) { T t = TANH(x); *out = (T)1 - t * t; } else *out = 0; return 0; }  /* ops.h:72-75 */ \
    case 13: { T ex = M(pow)((T)M_E, x); *out = (ex * (x + ex + (T)1)) / M(pow)(ex + (T)1, (T)2); return 0; } /* ops.h:993-996 */ \
    case 14: *out = (T)1 / (M(sqrt)(x - (T)1) * M(sqrt)(x + (T)1)); return 0;  /* ops.h:159-160 */           \
    case 15: *out = (T)1 / M(sqrt)(M(pow)(x, (T)2) + (T)1); return 0;          /* ops.h:155-156 */           \
    case 16: *out = M(cosh)(x); return 0;                                      /* ops.h:1048 */              \
    case 17: *out = (T)1 / (M(exp)(x) + (T)1); return 0;                       /* ops.h:1042-1045 */         \
    case 18: *out = x * ((T)1 - x); return 0;                                  /* ops.h:1167 */              \
    case 21: *out = (T)3 * x * x; return 0;                                    /* ops.h:1166 */              \
    case 30: *out = M(acos)(x); return 0;                                      /* ops.h:363-365 */           \
    case 31: *out = M(asin)(x); return 0;                                                                     \
    case 32: *out = M(atan)(x); return 0;                                                                     \
    case 33: *out = x < (T)-1 ? (T)-1 : x > (T)1 ? (T)1 : x; return 0;         /* ops.h:67-70 */             \
    case 34: *out = x / ((T)1 + M(fabs)(x)); return 0;                         /* templatemath.h:302-306 */  \
    case 36: { T v = (T)0.2f * x + (T)0.5f; v = v > 0 ? v : 0; *out = v < 1 ? v : 1; return 0; } /* ops.h:973-976 */ \
    case 37: {                                                                 /* ops.h:1065-1074 */         \
      T dis = ((T)2 / (T)3) * x;                                                                              \
      T sg = dis < 0 ? (T)-1 : dis > 0 ? (T)1 : (T)0;                                                         \
      T th = sg * ((T)1 - ((T)1 / ((T)1 + M(fabs)(dis) + M(pow)(dis, (T)2) + (T)1.41645f * M(pow)(dis, (T)4)))); \
      *out = (T)1.7159f * th; return 0;                                                                       \
    }                                                                                                         \
    case 38: { T t = TANH(x); *out = t > 0 ? t : 0; return 0; }                /* ops.h:1093-1095 */         \
    case 39: *out = M(sinh)(x); return 0;                                      /* ops.h:369-371 */           \
    case 40: *out = M(cosh)(x); return 0;                                                                     \
    case 41: *out = M(tan)(x); return 0;                                                                      \
    case 42: *out = x > (T)0 ? (T)SELU_L * x : (T)SELU_L * ((T)SELU_A * M(exp)(x) - (T)SELU_A); return 0; /* ops.h:978-982 */ \
    case 44: *out = M(log)(1 + x); return 0;                                   /* ops.h:375 */               \
    case 46: *out = M(acosh)(x); return 0;                                     /* ops.h:366-368 */           \
    case 47: *out = M(asinh)(x); return 0;                                                                    \
    case 48: *out = M(rint)(x); return 0;                                      /* ops.h:360 */               \
    case 49: *out = M(log)(SIGM(x)); return 0;                                 /* ops.h:1038-1040 */         \
    case 50: *out = M(erfc)(x); return 0;                                      /* ops.h:362 */               \
    case 51: *out = M(exp)(x) - (T)1; return 0;                                /* ops.h:378 */               \
    case 52: *out = M(atanh)(x); return 0;                                                                    \
    case 54: {                                                                 /* ops.h:1020-1025 */         \
      T x17 = (T)1.702f * x, ep = M(exp)(x17), o = (T)1 + ep;                                                 \
      *out = (ep * (o + x17)) / (o * o); return 0;                                                            \
    }                                                                                                         \
    case 56: {                                                                 /* ops.h:1027-1036 */         \
      T x79 = (T)0.797885 * x, t1 = (T)0.0356774 * x, x03 = t1 * t1 * t1;                                     \
      T x39 = (T)0.398942 * x, t2 = (T)0.0535161 * x, x05 = t2 * t2 * t2;                                     \
      T scz = (T)1 / M(cosh)(x79 + x03);                                                                      \
      *out = (T)0.5 + (x39 + x05) * (scz * scz) + (T)0.5 * TANH(x79 + x03); return 0;                         \
    }                                                                                                         \
    case 57: *out = x * TANH(M(log)((T)1 + M(exp)(x))); return 0;              /* ops.h:999-1001 */          \
    case 58: {                                                                 /* ops.h:1003-1008 */         \
      T ex = M(exp)(x), e2x = ex * ex, e3x = ex * ex * ex;                                                    \
      *out = (ex * (4 * (x + 1) + 4 * e2x + e3x + ex * (4 * x + 6))) / M(pow)(2 * ex + e2x + 2, (T)2); return 0; \
    }                                                                                                         \
    default: return 1;                                                                                        \
  }
#define MF(fn) fn##f
#define MD(fn) fn
static int strict_tail_f(int op, float x, float *out) { STRICT_TAIL(float, MF, ref_tanhf, ref_sigmoidf) }
static int strict_tail_d(int op, double x, double *out) { STRICT_TAIL(double, MD, ref_tanhd, ref_sigmoidd) }

/* TransformStrict opNums                      loops/legacy_ops.h:54-64; functors ops/ops.h:192-200,988-1019 */
static int strict_f(int op, float x, float *out) {
  switch (op) {
    case 22: *out = cosf(x); return 0;
    case 23: *out = expf(x); return 0;
    case 24: *out = logf(x); return 0;
    case 26: *out = ref_sigmoidf(x); return 0;
    case 27: *out = sinf(x); return 0;
    case 28: *out = logf(1.0f + expf(x)); return 0;                   /* SoftPlus  templatemath.h:272-274 */
    case 29: *out = ref_tanhf(x); return 0;
    case 43: *out = x * ref_sigmoidf(x); return 0;                    /* Swish     ops.h:988-990 */
    case 45: *out = erff(x); return 0;
    case 53: *out = x * ref_sigmoidf(1.702f * x); return 0;           /* GELU      ops.h:1010-1012 */
    case 55: {                                                        /* PreciseGELU ops.h:1015-1019 */
      float sp = sqrtf(2.0f / (float)M_PI);
      float xp = x + powf(0.044715f * x, 3.0f);
      *out = (x / 2.0f) * (1.0f + ref_tanhf(sp * xp));
      return 0;
    }
    default: return strict_tail_f(op, x, out);
  }
}
static int strict_d(int op, double x, double *out) {
  switch (op) {
    case 22: *out = cos(x); return 0;
    case 23: *out = exp(x); return 0;
    case 24: *out = log(x); return 0;
    case 26: *out = ref_sigmoidd(x); return 0;
    case 27: *out = sin(x); return 0;
    case 28: *out = log(1.0 + exp(x)); return 0;
    case 29: *out = ref_tanhd(x); return 0;
    case 43: *out = x * ref_sigmoidd(x); return 0;
    case 45: *out = erf(x); return 0;
    case 53: *out = x * ref_sigmoidd((double)1.702f * x); return 0;
    case 55: {
      double sp = sqrt(2.0 / M_PI);
      double xp = x + pow(0.044715 * x, 3.0);
      *out = (x / 2.0) * (1.0 + ref_tanhd(sp * xp));
      return 0;
    }
    default: return strict_tail_d(op, x, out);
  }
}

/* ---------------------------------------------------------------------------------------------
 * execTransformStrict / execTransformFloat    legacy/cpu/NativeOps.cpp:2280-2297, :2202-2219
 *   -> NativeOpExecutioner_transform.cpp:27-42,115-131 -> helpers/Loops.h:1080-1199
 * z[off_z(i)] = Op(x[off_x(i)]); extra params are ignored for same-type transforms (Loops.h:1178-1180).
 * The reference silently skips elements whose strided offset is >= length (Loops.h:1144-1153); this
 * restatement visits every element instead (documented divergence for views).
 * ------------------------------------------------------------------------------------------- */
int orc_transform_strict(int opNum, const void *x, const int64_t *xsi, void *z, const int64_t *zsi) {
  int xdt = orc_dtype(xsi), zdt = orc_dtype(zsi);
  if (xdt != zdt || !dt_is_float(xdt)) return 2;
  int64_t n = orc_length(xsi);
  if (n != orc_length(zsi)) return 3;
  float probe_f; double probe_d;
  if (strict_f(opNum, 0.5f, &probe_f) || strict_d(opNum, 0.5, &probe_d)) return 1;
  PAR_FOR
  for (int64_t i = 0; i < n; i++) {
    int64_t xo = orc_offset(xsi, i), zo = orc_offset(zsi, i);
    if (xdt == ORC_DOUBLE) {
      double r = 0; strict_d(opNum, ((const double *)x)[xo], &r); ((double *)z)[zo] = r;
    } else {
      float r = 0; strict_f(opNum, ldf(x, xdt, xo), &r); st(z, zdt, zo, r);
    }
  }
  return 0;
}

/* TransformFloat: 1 Sqrt, 3 RSqrt             loops/legacy_ops.h:67; ops/ops.h:2200-2205 */
int orc_transform_float(int opNum, const void *x, const int64_t *xsi, void *z, const int64_t *zsi) {
  int xdt = orc_dtype(xsi), zdt = orc_dtype(zsi);
  if (!dt_is_float(zdt)) return 2;
  if (opNum != 1 && opNum != 3) return 1;
  int64_t n = orc_length(xsi);
  if (n != orc_length(zsi)) return 3;
  PAR_FOR
  for (int64_t i = 0; i < n; i++) {
    int64_t xo = orc_offset(xsi, i), zo = orc_offset(zsi, i);
    if (zdt == ORC_DOUBLE) {
      double s = sqrt(ld(x, xdt, xo));
      ((double *)z)[zo] = opNum == 1 ? s : 1.0 / s;
    } else {
      /* sd_sqrt<X,Z>: cast to Z first, sqrt in Z (templatemath.h:1175-1180) */
      float s = rnd(sqrtf(rnd(ldf(x, xdt, xo), zdt)), zdt);
      st(z, zdt, zo, opNum == 1 ? s : 1.0f / s);
    }
  }
  return 0;
}

/* TransformSame: loops/legacy_ops.h:40-44; functors ops/ops.h:192-207,359,481,1165.  1 Sign is declared through
 * DECLARE_UNARY_CONDITIONAL_OP with the sign expression (d1 > 0) - (d1 < 0) as the CONDITION and 1 / -1 as the values
 * (ops.h:217-219): 1 for every non-zero number, -1 for zero and NaN.  Not restated here: 13 CompareAndSetTransform and
 * 19 ClipByValue (extra parameters; oracle.py holds them). */
static int same_d(int op, double x, double *out) {
  switch (op) {
    case 0: *out = fabs(x); return 0;
    case 1: *out = ((x > 0.0) - (x < 0.0)) ? 1.0 : -1.0; return 0;
    case 2: *out = 1.0; return 0;
    case 3: *out = -x; return 0;
    case 4: *out = round(x); return 0;           /* p_round = round(): halves away from zero */
    case 5: *out = x * (1.0 - x); return 0;
    case 6: *out = x * x * x; return 0;
    case 7: *out = 1.0 - x; return 0;
    case 11: *out = 1.0 / x; return 0;
    case 12: *out = x * x; return 0;
    case 15: case 21: *out = x; return 0;
    case 17: *out = ceil(x); return 0;
    case 18: *out = floor(x); return 0;
    default: return 1;
  }
}
static int same_f(int op, float x, float *out) {
  switch (op) {
    case 0: *out = fabsf(x); return 0;
    case 1: *out = ((x > 0.0f) - (x < 0.0f)) ? 1.0f : -1.0f; return 0;
    case 2: *out = 1.0f; return 0;
    case 3: *out = -x; return 0;
    case 4: *out = roundf(x); return 0;
    case 5: *out = x * (1.0f - x); return 0;
    case 6: *out = x * x * x; return 0;
    case 7: *out = 1.0f - x; return 0;
    case 11: *out = 1.0f / x; return 0;
    case 12: *out = x * x; return 0;
    case 15: case 21: *out = x; return 0;
    case 17: *out = ceilf(x); return 0;
    case 18: *out = floorf(x); return 0;
    default: return 1;
  }
}
int orc_transform_same(int opNum, const void *x, const int64_t *xsi, void *z, const int64_t *zsi) {
  int xdt = orc_dtype(xsi), zdt = orc_dtype(zsi);
  if (xdt != zdt || !dt_is_float(xdt)) return 2;
  int64_t n = orc_length(xsi);
  if (n != orc_length(zsi)) return 3;
  double pd; if (same_d(opNum, 0.5, &pd)) return 1;
  PAR_FOR
  for (int64_t i = 0; i < n; i++) {
    int64_t xo = orc_offset(xsi, i), zo = orc_offset(zsi, i);
    if (xdt == ORC_DOUBLE) {
      double r = 0; same_d(opNum, ((const double *)x)[xo], &r); ((double *)z)[zo] = r;
    } else {
      float r = 0; same_f(opNum, ldf(x, xdt, xo), &r); st(z, zdt, zo, r);
    }
  }
  return 0;
}

/* ---------------------------------------------------------------------------------------------
 * execPairwiseTransform                       legacy/cpu/NativeOps.cpp:1238-1282
 *   -> NativeOpExecutioner_pairwise_floats.cpp:23-68 -> loops/cpu/pairwise.hpp:87-169
 * z[i] = op(x[i], y[i]) over equal lengths, every operand through its own shapeInfo walk; x or y must
 * carry z's dtype.  opNums loops/legacy_ops.h:121-129; functors ops/ops.h:56-64,103-116,170-175,312-317.
 * The reference applies x->offset() twice for views (NativeOps.cpp:1245-1257 on top of buffer());
 * this restatement, like the product, applies it once.
 * ------------------------------------------------------------------------------------------- */
/* Binary functors by name, shared by the three tables below (ops/ops.h lines beside each). */
enum {
  B_ADD, B_COPY, B_DIV, B_MUL, B_RSUB, B_SUB, B_MAX, B_MIN, B_RDIV, B_SQSUB, B_POW, B_REMAINDER, B_FMOD, B_ATAN2,
  B_TRUNCDIV, B_FLOORDIV, B_FLOORMOD, B_REVMOD, B_SAFEDIV, B_MOD, B_LOR, B_LXOR, B_LNOT, B_LAND, B_AMAX, B_AMIN,
  B_TRUNCMOD, B_REPLACENANS, B_ELU, B_ELU_D, B_LRELU, B_LRELU_D, B_LOGX, B_RELU, B_RELU6, B_RELU_D, B_STEP,
  B_LSTMCLIP, B_SQRSUB, B_REVPOW, B_SXE, B_NONE
};
#define BINARY_BODY(T, M)                                                                                      \
  switch (fn) {                                                                                                \
    case B_ADD: return a + b;                              /* ops.h:56 */                                      \
    case B_COPY: return b;                                 /* ops.h:312-317 */                                 \
    case B_DIV: return a / b;                                                                                  \
    case B_MUL: return a * b;                                                                                  \
    case B_RSUB: return b - a;                             /* ops.h:63 */                                      \
    case B_SUB: return a - b;                                                                                  \
    case B_MAX: return a > b ? a : b;                      /* ops.h:103-108 */                                 \
    case B_MIN: return a < b ? a : b;                                                                          \
    case B_RDIV: return b / a;                             /* ops.h:64 */                                      \
    case B_SQSUB: { T d = a - b; return d * d; }           /* ops.h:174 */                                     \
    case B_POW: return M(pow)(a, b);                       /* ops.h:165 */                                     \
    case B_REMAINDER: return M(remainder)(a, b);           /* ops.h:228 */                                     \
    case B_FMOD: return M(fmod)(a, b);                     /* ops.h:229 */                                     \
    case B_ATAN2: return M(atan2)(a, b);                   /* ops.h:79; templatemath.h:321-324 */              \
    case B_TRUNCDIV: return (int)b == 0 ? (T)0 : (T)((int)a / (int)b);   /* ops.h:240-245; a zero divisor traps there */ \
    case B_FLOORDIV: return (T)floor((double)a / (double)b);   /* op_macros_special.h:87-93 */                 \
    case B_FLOORMOD: {                                     /* ops.h:260-267 */                                 \
      T m = M(fmod)(a, b);                                                                                     \
      return ((a < 0) == (b < 0)) ? m : M(fmod)(m + b, b);                                                     \
    }                                                                                                          \
    case B_REVMOD: return (int)a == 0 ? (T)0 : (T)((int)b % (int)a);     /* ops.h:1747-1752 */                 \
    case B_SAFEDIV: return b == 0 ? (T)0 : a / b;          /* ops.h:232-233 */                                 \
    case B_MOD: return a - M(floor)(a / b) * b;            /* ops.h:1708-1715 */                               \
    case B_LOR: return (T)((int)a | (int)b);               /* ops.h:2423-2428 */                               \
    case B_LXOR: return (T)(((int)a | (int)b) & ~((int)a & (int)b));                                           \
    case B_LNOT: return (T)(!((int)a && (int)b));                                                              \
    case B_LAND: return (T)((int)a & (int)b);                                                                  \
    case B_AMAX: return M(fabs)(a) > M(fabs)(b) ? a : b;   /* ops.h:89-101 */                                  \
    case B_AMIN: return M(fabs)(a) < M(fabs)(b) ? a : b;                                                       \
    case B_TRUNCMOD: return (int)b == 0 ? (T)0 : (T)((int)a % (int)b);   /* ops.h:247-252 */                   \
    case B_REPLACENANS: return isnan(a) ? b : a;           /* ops.h:582-587 */                                 \
    case B_ELU: return a >= 0 ? a : b * (M(exp)(a) - (T)1);    /* templatemath.h:233-240 */                    \
    case B_ELU_D: return a >= 0 ? (T)1 : b * M(exp)(a);        /* templatemath.h:255-262 */                    \
    case B_LRELU: return a < 0 ? b * a : a;                /* ops.h:1127-1131 */                               \
    case B_LRELU_D: return a >= 0 ? (T)1 : b;              /* ops.h:1133-1138 */                               \
    case B_LOGX: return M(log)(a) / M(log)(b);             /* ops.h:144-149 */                                 \
    case B_RELU: return a < b ? b : a;                     /* ops.h:1108-1112 */                               \
    case B_RELU6: { T r = a < b ? b : a; return r < 6 ? r : (T)6; }                                            \
    case B_RELU_D: return a > b ? (T)1 : (T)0;                                                                 \
    case B_STEP: return a > b ? (T)1 : (T)0;               /* ops.h:347-350 */                                 \
    case B_LSTMCLIP: return a > b ? b : a < -b ? -b : a;   /* ops.h:337-345 */                                 \
    case B_SQRSUB: { T d = b - a; return d * d; }          /* op_macros_special.h:820-827 */                   \
    case B_REVPOW: return M(pow)(b, a);                    /* ops.h:166 */                                     \
    case B_SXE: return a * ((T)1 - b) + (T)0.5f * b;       /* ops.h:352-355 */                                 \
    default: return a;                                                                                         \
  }
static float bin_f(int fn, float a, float b) { BINARY_BODY(float, MF) }
static double bin_d(int fn, double a, double b) { BINARY_BODY(double, MD) }
/* loops/legacy_ops.h:121-129 */
static int pairwise_fn(int op) {
  switch (op) {
    case 0: return B_ADD; case 1: return B_COPY; case 2: return B_DIV; case 3: return B_MUL; case 4: return B_POW;
    case 5: return B_RSUB; case 6: return B_SUB; case 7: return B_MAX; case 8: return B_MIN; case 9: return B_COPY;
    case 11: return B_RDIV; case 14: return B_REMAINDER; case 15: return B_FMOD; case 16: return B_ATAN2;
    case 17: return B_TRUNCDIV; case 18: return B_FLOORDIV; case 19: return B_FLOORMOD; case 20: return B_SQSUB;
    case 21: return B_REVMOD; case 22: return B_SAFEDIV; case 23: return B_MOD; case 27: return B_LOR;
    case 28: return B_LXOR; case 29: return B_LNOT; case 30: return B_LAND; case 34: return B_AMAX;
    case 35: return B_AMIN; case 36: return B_TRUNCMOD; case 37: return B_REPLACENANS; case 38: return B_SAFEDIV;
    default: return B_NONE;
  }
}
/* loops/legacy_ops.h:78-86 */
static int scalar_fn(int op) {
  switch (op) {
    case 0: return B_ADD; case 1: return B_SUB; case 2: return B_MUL; case 3: return B_DIV; case 4: return B_RDIV;
    case 5: return B_RSUB; case 6: return B_MAX; case 7: return B_ELU; case 8: return B_ELU_D; case 13: return B_MIN;
    case 14: return B_COPY; case 15: return B_MOD; case 16: return B_REVMOD; case 17: return B_REMAINDER;
    case 18: return B_FMOD; case 19: return B_TRUNCDIV; case 20: return B_FLOORDIV; case 21: return B_FLOORMOD;
    case 22: return B_SQSUB; case 23: return B_SAFEDIV; case 24: return B_AMAX; case 25: return B_AMIN;
    case 26: return B_ATAN2; case 27: return B_LOR; case 28: return B_LXOR; case 29: return B_LNOT; case 30: return B_LAND;
    case 31: return B_POW; case 34: return B_SXE; case 35: return B_LRELU; case 36: return B_LRELU_D;
    case 37: return B_REPLACENANS; case 38: return B_LOGX; case 39: return B_RELU; case 40: return B_RELU6;
    case 41: return B_STEP; case 42: return B_LSTMCLIP; case 43: return B_TRUNCMOD; case 44: return B_SQRSUB;
    case 45: return B_REVPOW; case 46: return B_SAFEDIV; case 49: return B_RELU_D;
    default: return B_NONE;
  }
}
/* loops/legacy_ops.h:34-39 */
static int broadcast_fn(int op) {
  switch (op) {
    case 0: return B_ADD; case 1: return B_SUB; case 2: return B_MUL; case 3: return B_DIV; case 4: return B_RDIV;
    case 5: return B_RSUB; case 6: return B_COPY; case 7: return B_POW; case 13: return B_MIN; case 14: return B_MAX;
    case 15: return B_AMIN; case 16: return B_AMAX; case 17: return B_SQSUB; case 18: return B_FLOORMOD;
    case 19: return B_FLOORDIV; case 20: return B_REVMOD; case 21: return B_SAFEDIV; case 22: return B_MOD;
    case 23: return B_TRUNCDIV; case 26: return B_ATAN2; case 27: return B_LOR; case 28: return B_LXOR;
    case 29: return B_LNOT; case 30: return B_LAND; case 31: return B_SAFEDIV;
    default: return B_NONE;
  }
}

static inline int pw_d(int op, double a, double b, double *r) {
  switch (op) {
    case 0: *r = a + b; return 0;
    case 1: *r = b; return 0;               /* CopyPws */
    case 2: *r = a / b; return 0;
    case 3: *r = a * b; return 0;
    case 5: *r = b - a; return 0;           /* ReverseSubtract */
    case 6: *r = a - b; return 0;
    case 7: *r = a > b ? a : b; return 0;   /* MaxPairwise (sd_max) */
    case 8: *r = a < b ? a : b; return 0;   /* MinPairwise */
    case 11: *r = b / a; return 0;          /* ReverseDivide */
    case 20: *r = (a - b) * (a - b); return 0; /* SquaredSubtract */
    default: { int fn = pairwise_fn(op); if (fn == B_NONE) return 1; *r = bin_d(fn, a, b); return 0; }
  }
}
static inline int pw_f(int op, float a, float b, float *r) {
  switch (op) {
    case 0: *r = a + b; return 0;
    case 1: *r = b; return 0;
    case 2: *r = a / b; return 0;
    case 3: *r = a * b; return 0;
    case 5: *r = b - a; return 0;
    case 6: *r = a - b; return 0;
    case 7: *r = a > b ? a : b; return 0;
    case 8: *r = a < b ? a : b; return 0;
    case 11: *r = b / a; return 0;
    case 20: { float d = a - b; *r = d * d; return 0; }
    default: { int fn = pairwise_fn(op); if (fn == B_NONE) return 1; *r = bin_f(fn, a, b); return 0; }
  }
}
int orc_pairwise(int opNum, const void *x, const int64_t *xsi, const void *y, const int64_t *ysi, void *z,
                 const int64_t *zsi) {
  int xdt = orc_dtype(xsi), ydt = orc_dtype(ysi), zdt = orc_dtype(zsi);
  if (xdt != zdt && ydt != zdt) return 2; /* NativeOpExecutioner_pairwise_floats.cpp:34,46 */
  if (!dt_is_float(zdt)) return 2;
  int64_t n = orc_length(zsi);
  if (orc_length(xsi) != n || orc_length(ysi) != n) return 3;
  double pd; if (pw_d(opNum, 1, 1, &pd)) return 1;
  PAR_FOR
  for (int64_t i = 0; i < n; i++) {
    int64_t xo = orc_offset(xsi, i), yo = orc_offset(ysi, i), zo = orc_offset(zsi, i);
    if (zdt == ORC_DOUBLE) {
      double r = 0; pw_d(opNum, ld(x, xdt, xo), ld(y, ydt, yo), &r); ((double *)z)[zo] = r;
    } else {
      /* operands are cast to Z before the arithmetic (sd_add<X,Y,Z> etc.) */
      float r = 0; pw_f(opNum, rnd(ldf(x, xdt, xo), zdt), rnd(ldf(y, ydt, yo), zdt), &r); st(z, zdt, zo, r);
    }
  }
  return 0;
}

/* ---------------------------------------------------------------------------------------------
 * execScalar                                   legacy/cpu/NativeOps.cpp (execScalar) -> loops/cpu/scalar.hpp
 * z[i] = op(x[i], scalar, params) for every element, x and z through their own shapeInfo; the scalar is held
 * in an array of x's type, so it is rounded to that type first.  opNums loops/legacy_ops.h:78-86.
 * ------------------------------------------------------------------------------------------- */
int orc_scalar(int opNum, const void *x, const int64_t *xsi, double scalar, void *z, const int64_t *zsi) {
  int xdt = orc_dtype(xsi), zdt = orc_dtype(zsi);
  if (xdt != zdt || !dt_is_float(xdt)) return 2;
  int64_t n = orc_length(xsi);
  if (n != orc_length(zsi)) return 3;
  int fn = scalar_fn(opNum);
  if (fn == B_NONE) return 1;
  float sf = rnd((float)scalar, xdt);
  PAR_FOR
  for (int64_t i = 0; i < n; i++) {
    int64_t xo = orc_offset(xsi, i), zo = orc_offset(zsi, i);
    if (xdt == ORC_DOUBLE) ((double *)z)[zo] = bin_d(fn, ((const double *)x)[xo], scalar);
    else st(z, zdt, zo, bin_f(fn, ldf(x, xdt, xo), sf));
  }
  return 0;
}

/* ---------------------------------------------------------------------------------------------
 * execBroadcast                                loops/cpu/broadcasting.hpp (exec over TADs)
 * x is cut into TADs along `dims`; y has the TAD's length; z_tad[i] = op(x_tad[i], y[i]) for every TAD.
 * opNums loops/legacy_ops.h:34-39.  z must have x's shape; here z's TADs are taken with the same dims.
 * ------------------------------------------------------------------------------------------- */
int orc_broadcast(int opNum, const void *x, const int64_t *xsi, const void *y, const int64_t *ysi, void *z,
                  const int64_t *zsi, const int64_t *dims, int ndims) {
  int xdt = orc_dtype(xsi), ydt = orc_dtype(ysi), zdt = orc_dtype(zsi);
  if (xdt != zdt || ydt != zdt || !dt_is_float(zdt)) return 2;
  int fn = broadcast_fn(opNum);
  if (fn == B_NONE) return 1;
  int64_t n = orc_length(xsi);
  if (n != orc_length(zsi)) return 3;
  int64_t xtad[2 * ORC_MAX_RANK + 4], ztad[2 * ORC_MAX_RANK + 4];
  int64_t ntads = orc_tad(xsi, dims, ndims, xtad, NULL);
  if (ntads <= 0) return 3;
  int64_t *xoff = (int64_t *)malloc(sizeof(int64_t) * (size_t)ntads), *zoff = (int64_t *)malloc(sizeof(int64_t) * (size_t)ntads);
  orc_tad(xsi, dims, ndims, xtad, xoff);
  orc_tad(zsi, dims, ndims, ztad, zoff);
  int64_t tadLen = orc_length(xtad);
  if (tadLen != orc_length(ysi)) { free(xoff); free(zoff); return 3; }
  for (int64_t t = 0; t < ntads; t++) {
    for (int64_t i = 0; i < tadLen; i++) {
      int64_t xo = xoff[t] + orc_offset(xtad, i), zo = zoff[t] + orc_offset(ztad, i), yo = orc_offset(ysi, i);
      if (zdt == ORC_DOUBLE) ((double *)z)[zo] = bin_d(fn, ((const double *)x)[xo], ((const double *)y)[yo]);
      else st(z, zdt, zo, bin_f(fn, ldf(x, xdt, xo), ldf(y, ydt, yo)));
    }
  }
  free(xoff); free(zoff);
  return 0;
}

/* ---------------------------------------------------------------------------------------------
 * reductions
 * dims handling: the facade normalises negative dims (legacy/cpu/NativeOps.cpp:1704-1711) and turns them
 * into [kept dims.., reduced dims..] (helpers/impl/ShapeUtils.cpp:1305-1327); loops run kept dims as the
 * outer walk and reduced dims as the inner, sequential accumulate in InterType (helpers/Loops.h:153-199).
 * z is written through its own shapeInfo in row-major order of the kept dims (unit dims of a keepDims z
 * collapse, NativeOps.cpp:1716-1720).
 * ------------------------------------------------------------------------------------------- */
typedef struct {
  int orank, irank;
  int64_t oshape[ORC_MAX_RANK], ostride[ORC_MAX_RANK], ishape[ORC_MAX_RANK], istride[ORC_MAX_RANK];
  int64_t olen, ilen;
} RedPlan;

static int red_plan(const int64_t *xsi, const int64_t *dims, int ndims, RedPlan *p) {
  int r = si_rank(xsi), red[ORC_MAX_RANK] = {0};
  if (ndims == 0 || (ndims == 1 && dims[0] == 2147483647)) { for (int i = 0; i < r; i++) red[i] = 1; }
  for (int i = 0; i < ndims; i++) {
    if (dims[i] == 2147483647) continue;
    int64_t d = dims[i] < 0 ? dims[i] + r : dims[i];
    if (d < 0 || d >= r) return 1;
    red[d] = 1;
  }
  p->orank = p->irank = 0; p->olen = p->ilen = 1;
  for (int i = 0; i < r; i++) {
    if (red[i]) { p->ishape[p->irank] = si_shape(xsi)[i]; p->istride[p->irank++] = si_stride(xsi)[i]; p->ilen *= si_shape(xsi)[i]; }
    else { p->oshape[p->orank] = si_shape(xsi)[i]; p->ostride[p->orank++] = si_stride(xsi)[i]; p->olen *= si_shape(xsi)[i]; }
  }
  return 0;
}
static inline int64_t walk(int rank, const int64_t *shape, const int64_t *stride, int64_t idx) {
  int64_t off = 0;
  for (int i = rank - 1; i >= 0; i--) { off += (idx % shape[i]) * stride[i]; idx /= shape[i]; }
  return off;
}

/* ReduceSame: 0 Sum 1 Max 2 Min 3 Prod 4 ASum 5 AMax 6 AMin   loops/legacy_ops.h:100-101; ops/ops.h:2363-2368,1170-1243
 * ReduceFloat: 0 Mean 1 AMean 2 Norm1 3 Norm2 4 NormMax 7 SquaredNorm 8 Entropy 9 LogEntropy 10 ShannonEntropy
 *   legacy_ops.h:103-105; ops.h:2370-2378,1217-1298,1956-1973,2147-2153
 * accumulator type = float for float/half/bf16 (InterType, ops/op_types.h:213-226), double for double; the ReduceFloat
 * ops take it from Z (op_macros_reduce.h:778-782), and X may be any numeric type there
 * (NativeOpExecutioner_reduce.cpp:34-37,104-106: SD_NUMERIC_TYPES x SD_FLOAT_TYPES). */
#define RED_BODY(ACC_T, LOAD, ABS, SQRT, INF, LOG, LOG2, RX, RZ)                                                        \
  ACC_T s;                                                                                              \
  switch (kind) {                                                                                       \
    case 1: s = -INF; break;                                                                            \
    case 2: s = INF; break;                                                                             \
    case 3: s = 1; break;                                                                               \
    case 5: case 6: s = ABS(LOAD(0)); break; /* AMax/AMin start from |x[0]| (input[0], then abs'ed) */  \
    default: s = 0;                                                                                     \
  }                                                                                                     \
  for (int64_t j = 0; j < p.ilen; j++) {                                                                \
    ACC_T v = LOAD(j);                                                                                  \
    switch (kind) {                                                                                     \
      case 0: case 10: s = v + s; break;                                                                \
      case 1: s = v > s ? v : s; break;                                                                 \
      case 2: s = v < s ? v : s; break;                                                                 \
      case 3: s = v * s; break;                                                                         \
      case 4: case 11: case 12: s = ABS(v) + s; break;                                                  \
      case 5: case 14: s = ABS(v) > s ? ABS(v) : s; break;                                              \
      case 6: s = ABS(v) < s ? ABS(v) : s; break;                                                       \
      case 13: case 17: s = v * v + s; break;                                                           \
      /* Entropy / LogEntropy: x * log(x), the log taken in x's own type (ops.h:1966-1973,2147-2153) */ \
      case 18: case 19: s = v * RX(LOG(v)) + s; break;                                                  \
      /* ShannonEntropy: p * log2(p), the product formed in z's type (ops.h:1956-1963) */              \
      case 20: s = RZ(v * RX(LOG2(v))) + s; break;                                                      \
    }                                                                                                   \
  }                                                                                                     \
  switch (kind) {                                                                                       \
    case 10: case 11: s = s / (ACC_T)p.ilen; break;                                                     \
    case 13: s = SQRT(s); break;                                                                        \
    case 18: case 20: s = -s; break;                                                                    \
    /* sd_log<InterType, Z>(-reduction): this logarithm is the accumulator type's (ops.h:1966-1973) */  \
    case 19: s = sizeof(ACC_T) == 8 ? (ACC_T)log((double)-s) : (ACC_T)logf((float)-s); break;           \
  }

static int reduce_impl(int kind, const void *x, const int64_t *xsi, void *z, const int64_t *zsi, const int64_t *dims,
                       int ndims) {
  RedPlan p;
  if (red_plan(xsi, dims, ndims, &p)) return 3;
  int xdt = orc_dtype(xsi), zdt = orc_dtype(zsi);
  if (orc_length(zsi) != p.olen) return 3;
  /* z walk: strip unit dims so a keepDims z lines up with the kept dims */
  int64_t zshape[ORC_MAX_RANK], zstride[ORC_MAX_RANK]; int zr = 0;
  for (int i = 0; i < si_rank(zsi); i++)
    if (si_shape(zsi)[i] != 1) { zshape[zr] = si_shape(zsi)[i]; zstride[zr++] = si_stride(zsi)[i]; }
  PAR_FOR
  for (int64_t o = 0; o < p.olen; o++) {
    int64_t base = walk(p.orank, p.oshape, p.ostride, o);
    int64_t zo = walk(zr, zshape, zstride, o);
    if (kind >= 10 ? zdt == ORC_DOUBLE : xdt == ORC_DOUBLE) {
#define LOADD(j) (ld(x, xdt, base + walk(p.irank, p.ishape, p.istride, (j))))
#define NOROUND(v) (v)
/* the logarithm is taken in X's own type whatever the accumulator is (sd_log<X, Z> casts p_log<X>'s result, templatemath.h:287-299) */
#define LOGX(v) (xdt == ORC_DOUBLE ? log(v) : (double)rnd(logf((float)(v)), xdt))
#define LOG2X(v) (xdt == ORC_DOUBLE ? log2(v) : (double)rnd(log2f((float)(v)), xdt))
      RED_BODY(double, LOADD, fabs, sqrt, INFINITY, LOGX, LOG2X, NOROUND, NOROUND)
      st(z, zdt, zo, s);
    } else {
#define LOADF(j) (ldf(x, xdt, base + walk(p.irank, p.ishape, p.istride, (j))))
#define RNDX(v) rnd((v), xdt)
#define RNDZ(v) rnd((v), zdt)
      RED_BODY(float, LOADF, fabsf, sqrtf, INFINITY, logf, log2f, RNDX, RNDZ)
      st(z, zdt, zo, s);
    }
  }
  return 0;
}

/* execReduceSame / execReduceSame2            legacy/cpu/NativeOps.cpp:1330-1374,1687-1786
 *   -> NativeOpExecutioner_reduce.cpp:42-52 -> loops/cpu/reduce/reduce_same.hpp:39-106,156-193 */
int orc_reduce_same(int opNum, const void *x, const int64_t *xsi, void *z, const int64_t *zsi, const int64_t *dims,
                    int ndims) {
  if (opNum < 0 || opNum > 6) return 1;
  if (orc_dtype(xsi) != orc_dtype(zsi) || !dt_is_float(orc_dtype(xsi))) return 2;
  return reduce_impl(opNum, x, xsi, z, zsi, dims, ndims);
}
/* execReduceFloat / execReduceFloat2          legacy/cpu/NativeOps.cpp:1284-1328,1488-1584
 *   -> NativeOpExecutioner_reduce.cpp:98-120 -> loops/cpu/reduce/reduce_float.hpp:79-175,220-289 */
int orc_reduce_float(int opNum, const void *x, const int64_t *xsi, void *z, const int64_t *zsi, const int64_t *dims,
                     int ndims) {
  if (!dt_is_float(orc_dtype(zsi)) || dt_size(orc_dtype(xsi)) == 0) return 2;
  switch (opNum) {
    case 0: return reduce_impl(10, x, xsi, z, zsi, dims, ndims);
    case 1: return reduce_impl(11, x, xsi, z, zsi, dims, ndims);
    case 2: return reduce_impl(12, x, xsi, z, zsi, dims, ndims);
    case 3: return reduce_impl(13, x, xsi, z, zsi, dims, ndims);
    case 4: return reduce_impl(14, x, xsi, z, zsi, dims, ndims);
    case 7: return reduce_impl(17, x, xsi, z, zsi, dims, ndims);
    case 8: return reduce_impl(18, x, xsi, z, zsi, dims, ndims);   /* Entropy */
    case 9: return reduce_impl(19, x, xsi, z, zsi, dims, ndims);   /* LogEntropy */
    case 10: return reduce_impl(20, x, xsi, z, zsi, dims, ndims);  /* ShannonEntropy */
    default: return 1;
  }
}

/* ---------------------------------------------------------------------------------------------
 * execSummaryStatsScalar / execSummaryStatsTad   legacy/cpu/NativeOps.cpp:2167-2200 -> loops/cpu/summarystatsreduce.cpp
 * per output: SummaryStatsData {n, mean, M2} in double, fed one element at a time (Welford's update, the form
 * loops/summarystatsreduce.h:190-211 takes for a one-element right-hand side); variance = M2 / n (0 for n <= 1),
 * bias-corrected M2 / (n - 1) unless that is negative (ops/ops.h:2157-2190); opNum 0 variance, 1 standard deviation.
 * ------------------------------------------------------------------------------------------- */
int orc_summary_stats(int opNum, const void *x, const int64_t *xsi, void *z, const int64_t *zsi, const int64_t *dims, int ndims,
                      int biasCorrected) {
  if (opNum != 0 && opNum != 1) return 1;
  RedPlan p;
  if (red_plan(xsi, dims, ndims, &p)) return 3;
  int xdt = orc_dtype(xsi), zdt = orc_dtype(zsi);
  if (!dt_is_float(zdt)) return 2;
  if (orc_length(zsi) != p.olen) return 3;
  int64_t zshape[ORC_MAX_RANK], zstride[ORC_MAX_RANK]; int zr = 0;
  for (int i = 0; i < si_rank(zsi); i++)
    if (si_shape(zsi)[i] != 1) { zshape[zr] = si_shape(zsi)[i]; zstride[zr++] = si_stride(zsi)[i]; }
  for (int64_t o = 0; o < p.olen; o++) {
    int64_t base = walk(p.orank, p.oshape, p.ostride, o);
    double n = 0, mean = 0, m2 = 0;
    for (int64_t j = 0; j < p.ilen; j++) {
      double v = ld(x, xdt, base + walk(p.irank, p.ishape, p.istride, j));
      n += 1.0;
      double delta = v - mean;
      mean += delta / n;
      m2 += delta * (v - mean);
    }
    double var = n <= 1.0 ? 0.0 : m2 / n;
    if (biasCorrected) { double c = n <= 1.0 ? 0.0 : m2 / (n - 1.0); if (!(c < 0.0)) var = c; }
    st(z, zdt, walk(zr, zshape, zstride, o), opNum == 1 ? sqrt(var) : var);
  }
  return 0;
}

/* execReduceLong (0 CountNonZero, 1 CountZero: ops/ops.h:1180-1198) and execReduceBool (0 Any: the sum of the elements is
 * positive, 1 All: no element is zero; ops/ops.h:1200-1215).  kind: 0/1 = long ops, 10/11 = bool ops. */
int orc_reduce_count(int kind, const void *x, const int64_t *xsi, void *z, const int64_t *zsi, const int64_t *dims, int ndims) {
  RedPlan p;
  if (red_plan(xsi, dims, ndims, &p)) return 3;
  int xdt = orc_dtype(xsi), zdt = orc_dtype(zsi);
  if (orc_length(zsi) != p.olen) return 3;
  if ((kind < 10 && zdt != ORC_INT64) || (kind >= 10 && zdt != ORC_BOOL)) return 2;
  int64_t zshape[ORC_MAX_RANK], zstride[ORC_MAX_RANK]; int zr = 0;
  for (int i = 0; i < si_rank(zsi); i++)
    if (si_shape(zsi)[i] != 1) { zshape[zr] = si_shape(zsi)[i]; zstride[zr++] = si_stride(zsi)[i]; }
  for (int64_t o = 0; o < p.olen; o++) {
    int64_t base = walk(p.orank, p.oshape, p.ostride, o);
    double sum = 0; int64_t zeros = 0;
    for (int64_t j = 0; j < p.ilen; j++) {
      double v = ld(x, xdt, base + walk(p.irank, p.ishape, p.istride, j));
      sum += v;
      zeros += v == 0.0;
    }
    int64_t zo = walk(zr, zshape, zstride, o);
    switch (kind) {
      case 0: ((int64_t *)z)[zo] = p.ilen - zeros; break;
      case 1: ((int64_t *)z)[zo] = zeros; break;
      case 10: ((unsigned char *)z)[zo] = sum > 0.0; break;
      case 11: ((unsigned char *)z)[zo] = zeros == 0; break;
      default: return 1;
    }
  }
  return 0;
}

/* execReduce3 / execReduce3Scalar / execReduce3Tad   loops/cpu/reduce3.hpp; functors ops/ops.h:117-134,483-541
 * 0 Manhattan sum|x-y|, 1 Euclidean sqrt(sum (x-y)^2), 2 CosineSimilarity xy / (|x| |y|), 3 Dot, 5 CosineDistance 1 - cos,
 * 6 JaccardDistance 1 - sum min / sum max, 7 SimpleHamming (count x != y) / n.  Accumulated in double here.  The square root
 * of the Euclidean distance is what the reference's tests expect (NDArrayTests.cpp:1455-1488); the functor macro of this
 * snapshot leaves it out. */
int orc_reduce3(int opNum, const void *x, const int64_t *xsi, const void *y, const int64_t *ysi, void *z, const int64_t *zsi,
                const int64_t *dims, int ndims) {
  RedPlan p, py;
  if (red_plan(xsi, dims, ndims, &p) || red_plan(ysi, dims, ndims, &py)) return 3;
  if (p.olen != py.olen || p.ilen != py.ilen) return 3;
  int xdt = orc_dtype(xsi), ydt = orc_dtype(ysi), zdt = orc_dtype(zsi);
  if (!dt_is_float(zdt)) return 2;
  if (orc_length(zsi) != p.olen) return 3;
  if (opNum < 0 || opNum > 7 || opNum == 4) return 1;
  int64_t zshape[ORC_MAX_RANK], zstride[ORC_MAX_RANK]; int zr = 0;
  for (int i = 0; i < si_rank(zsi); i++)
    if (si_shape(zsi)[i] != 1) { zshape[zr] = si_shape(zsi)[i]; zstride[zr++] = si_stride(zsi)[i]; }
  for (int64_t o = 0; o < p.olen; o++) {
    int64_t xb = walk(p.orank, p.oshape, p.ostride, o), yb = walk(py.orank, py.oshape, py.ostride, o);
    double s0 = 0, s1 = 0, s2 = 0;
    for (int64_t j = 0; j < p.ilen; j++) {
      double u = ld(x, xdt, xb + walk(p.irank, p.ishape, p.istride, j));
      double v = ld(y, ydt, yb + walk(py.irank, py.ishape, py.istride, j));
      switch (opNum) {
        case 0: s0 += fabs(u - v); break;
        case 1: s0 += (u - v) * (u - v); break;
        case 2: case 5: s0 += u * v; s1 += u * u; s2 += v * v; break;
        case 3: s0 += u * v; break;
        case 6: s1 += u < v ? u : v; s2 += u > v ? u : v; break;
        case 7: s0 += u != v; break;
      }
    }
    double r = s0;
    switch (opNum) {
      case 1: r = sqrt(s0); break;
      case 2: r = s0 / (sqrt(s1) * sqrt(s2)); break;
      case 5: r = 1.0 - s0 / (sqrt(s1) * sqrt(s2)); break;
      case 6: r = 1.0 - s1 / s2; break;
      case 7: r = s0 / (double)p.ilen; break;
    }
    st(z, zdt, walk(zr, zshape, zstride, o), r);
  }
  return 0;
}

/* execTransformBool: loops/legacy_ops.h:49-51; predicates ops/ops.h:1140-1163,1927-1933; z is a BOOL array */
int orc_transform_bool(int opNum, const void *x, const int64_t *xsi, void *z, const int64_t *zsi) {
  int xdt = orc_dtype(xsi);
  if (orc_dtype(zsi) != ORC_BOOL || !dt_is_float(xdt)) return 2;
  int64_t n = orc_length(xsi);
  if (n != orc_length(zsi)) return 3;
  if (opNum < 1 || opNum > 8 || opNum == 5) return 1;
  for (int64_t i = 0; i < n; i++) {
    double v = ld(x, xdt, orc_offset(xsi, i));
    int r = 0;
    switch (opNum) {
      case 1: r = isinf(v); break;
      case 2: r = isnan(v); break;
      case 3: r = isfinite(v); break;
      case 4: r = !isfinite(v); break;
      case 6: r = v > 0; break;
      case 7: r = !(v != 0); break;     /* Not: !static_cast<bool>(d1) */
      case 8: r = v < 0; break;
    }
    ((unsigned char *)z)[orc_offset(zsi, i)] = r != 0;
  }
  return 0;
}

/* ---------------------------------------------------------------------------------------------
 * execIndexReduce / execIndexReduceScalar     legacy/cpu/NativeOps.cpp:1110-1170
 *   -> NativeOpExecutioner_indexreduce.cpp:20-46 -> loops/cpu/indexreduce.hpp:55-140
 *   -> helpers/cpu/loops/IndexReductionLoops.hpp:40-243
 * per TAD: start {value = start, index = 0}; replace iff strict compare holds, so the first extreme
 * wins, NaN is never selected and an all -inf row yields 0.  Index = row-major position inside the TAD.
 * opNums loops/legacy_ops.h:131-132; functors ops/op_macros_index_reduce.h:33-69, ops/ops.h:1977-2058,2383-2386.
 * The custom op argmax/argmin shares this contract (ops/declarable/helpers/cpu/indexReductions.hpp:176-210).
 * ------------------------------------------------------------------------------------------- */
int orc_index_reduce(int opNum, const void *x, const int64_t *xsi, void *z, const int64_t *zsi, const int64_t *dims,
                     int ndims) {
  if (opNum < 0 || opNum > 3) return 1;
  RedPlan p;
  if (red_plan(xsi, dims, ndims, &p)) return 3;
  int xdt = orc_dtype(xsi), zdt = orc_dtype(zsi);
  if (zdt != ORC_INT64 && zdt != ORC_INT32) return 2;
  if (orc_length(zsi) != p.olen) return 3;
  PAR_FOR
  for (int64_t o = 0; o < p.olen; o++) {
    int64_t base = walk(p.orank, p.oshape, p.ostride, o);
    double best;
    switch (opNum) { case 0: best = -INFINITY; break; case 1: best = INFINITY; break; case 2: best = 0; break; default: best = INFINITY; }
    int64_t bi = 0;
    for (int64_t j = 0; j < p.ilen; j++) {
      double v = ld(x, xdt, base + walk(p.irank, p.ishape, p.istride, j));
      int take;
      switch (opNum) {
        case 0: take = v > best; break;
        case 1: take = v < best; break;
        case 2: v = fabs(v); take = v > best; break;
        default: v = fabs(v); take = v < best; break;
      }
      if (take) { best = v; bi = j; }
    }
    /* z is written linearly: z[i] (IndexReductionLoops.hpp:61-75) */
    if (zdt == ORC_INT64) ((int64_t *)z)[o] = bi; else ((int32_t *)z)[o] = (int32_t)bi;
  }
  return 0;
}

/* ---------------------------------------------------------------------------------------------
 * top_k                                        ops/declarable/generic/parity_ops/top_k.cpp:31-57
 *   -> ops/declarable/helpers/cpu/top_k.cpp:34-125, restated literally, quirks included:
 *   k == 1: first maximum (strict <).  k > 1: the first k elements seed the candidate set; a later
 *   element enters only if it exceeds the current minimum AND equals no candidate (std::binary_search
 *   over the sorted copy), replacing the first candidate equal to that minimum.  needSort: values
 *   descending, and every position is re-derived as the LAST j with x[j] == value (so equal values
 *   share one position); else the candidates are ordered by their recorded positions (std::map).
 *   Values are compared as doubles (exact for every supported storage type).
 * ------------------------------------------------------------------------------------------- */
static int cmp_asc(const void *a, const void *b) { double x = *(const double *)a, y = *(const double *)b; return (x > y) - (x < y); }
int orc_top_k(const void *x, const int64_t *xsi, void *values, const int64_t *vsi, void *indices, const int64_t *isi,
              int64_t k, int needSort) {
  int r = si_rank(xsi), dt = orc_dtype(xsi), idt = orc_dtype(isi);
  if (r < 1) return 3;
  int64_t width = si_shape(xsi)[r - 1];
  if (k < 1 || k > width) return 3;
  if (idt != ORC_INT64 && idt != ORC_INT32) return 2;
  int64_t rows = orc_length(xsi) / width;
  const int64_t *xs = si_stride(xsi), *vs = si_stride(vsi), *is = si_stride(isi);
  double *top = (double *)malloc(sizeof(double) * (size_t)k), *sorted = (double *)malloc(sizeof(double) * (size_t)k);
  int64_t *tix = (int64_t *)malloc(sizeof(int64_t) * (size_t)k);
  for (int64_t e = 0; e < rows; e++) {
    int64_t xb = walk(r - 1, si_shape(xsi), xs, e), vb = walk(r - 1, si_shape(vsi), vs, e), ib = walk(r - 1, si_shape(isi), is, e);
#define XV(j) ld(x, dt, xb + (j) * xs[r - 1])
    if (k == 1) {
      int64_t maxPos = 0;
      double maxVal = XV(0);
      for (int64_t pos = 1; pos < width; pos++) if (maxVal < XV(pos)) { maxPos = pos; maxVal = XV(pos); }
      top[0] = maxVal; tix[0] = maxPos;
    } else {
      for (int64_t pos = 0; pos < k; pos++) { tix[pos] = pos; top[pos] = XV(pos); sorted[pos] = top[pos]; }
      qsort(sorted, (size_t)k, sizeof(double), cmp_asc);
      for (int64_t i = k; i < width; i++) {
        double val = XV(i), minTop = sorted[0];
        if (minTop < val) {
          int exists = 0;
          { int64_t lo = 0, hi = k; while (lo < hi) { int64_t mid = (lo + hi) / 2; if (sorted[mid] < val) lo = mid + 1; else hi = mid; }
            exists = lo < k && !(val < sorted[lo]); }
          if (!exists) {
            int64_t pos = 0;
            while (pos < k && top[pos] != sorted[0]) pos++;
            if (pos < k) { top[pos] = val; tix[pos] = i; }   /* std::find returning end() would write past the array */
            sorted[0] = val;
            qsort(sorted, (size_t)k, sizeof(double), cmp_asc);
          }
        }
      }
      if (needSort) {
        qsort(top, (size_t)k, sizeof(double), cmp_asc);
        for (int64_t a = 0, b = k - 1; a < b; a++, b--) { double tmp = top[a]; top[a] = top[b]; top[b] = tmp; }   /* descending */
        for (int64_t j = 0; j < width; j++) for (int64_t pos = 0; pos < k; pos++) if (top[pos] == XV(j)) tix[pos] = j;
      } else {
        /* std::map<index, value>: ascending positions, a repeated position keeps its last value */
        for (int64_t a = 1; a < k; a++) {
          int64_t ci = tix[a]; double cv = top[a]; int64_t b = a - 1;
          while (b >= 0 && tix[b] > ci) { tix[b + 1] = tix[b]; top[b + 1] = top[b]; b--; }
          tix[b + 1] = ci; top[b + 1] = cv;
        }
      }
    }
#undef XV
    for (int64_t pos = 0; pos < k; pos++) {
      if (values) st(values, dt, vb + pos * vs[r - 1], top[pos]);
      if (indices) { if (idt == ORC_INT64) ((int64_t *)indices)[ib + pos * is[r - 1]] = tix[pos]; else ((int32_t *)indices)[ib + pos * is[r - 1]] = (int32_t)tix[pos]; }
    }
  }
  free(top); free(sorted); free(tix);
  return 0;
}

/* ---------------------------------------------------------------------------------------------
 * softmax                                     ops/declarable/generic/nn/softmax.cpp:37-52
 *   -> ops/declarable/helpers/cpu/softmax.cpp:36-107 (vector), :252-353 (TAD loop / fallback)
 * same-shape-strict branch: max over finite values only (0 if none), inf/nan inputs mapped to
 * +-88 + max, diff = clamp(x - max, -88, 88), r = exp(diff), sum = max(sum r, 1e-6), out = r / sum.
 * fallback branch (in/out strides differ): max -> sub -> exp -> sum -> div with no clamp.
 * literal_half: carry max/sum/r in the storage type like the reference's `T sum` does.
 * ------------------------------------------------------------------------------------------- */
static int same_shape_strict(const int64_t *a, const int64_t *b) {
  if (si_rank(a) != si_rank(b)) return 0;
  for (int i = 0; i < 2 * si_rank(a); i++) if (a[1 + i] != b[1 + i]) return 0;
  return 1;
}
int orc_softmax(const void *x, const int64_t *xsi, void *z, const int64_t *zsi, int dim, int literal_half) {
  int r = si_rank(xsi), dt = orc_dtype(xsi);
  if (dt != orc_dtype(zsi) || !dt_is_float(dt)) return 2;
  if (dim < 0) dim += r;
  if (dim < 0 || dim >= r) return 3;
  int64_t n = orc_length(xsi);
  if (n != orc_length(zsi)) return 3;
  int isVector = 0; { int nontrivial = 0; for (int i = 0; i < r; i++) if (si_shape(xsi)[i] != 1) nontrivial++; isVector = nontrivial <= 1 && r <= 2 && r >= 1; }
  if (isVector && r != 1 && si_shape(xsi)[dim] == 1) { /* softmax.cpp:255-259 */
    for (int64_t i = 0; i < n; i++) st(z, dt, orc_offset(zsi, i), 1.0);
    return 0;
  }
  int64_t L = isVector ? n : si_shape(xsi)[dim];
  int64_t xs = isVector ? 0 : si_stride(xsi)[dim], zs = isVector ? 0 : si_stride(zsi)[dim];
  int clamp = isVector || same_shape_strict(xsi, zsi);
  /* outer walk over all dims except `dim` */
  int64_t oshape[ORC_MAX_RANK], oxs[ORC_MAX_RANK], ozs[ORC_MAX_RANK]; int orank = 0; int64_t olen = 1;
  if (!isVector)
    for (int i = 0; i < r; i++) if (i != dim) { oshape[orank] = si_shape(xsi)[i]; oxs[orank] = si_stride(xsi)[i]; ozs[orank++] = si_stride(zsi)[i]; olen *= si_shape(xsi)[i]; }
  const int lit = literal_half && (dt == ORC_HALF || dt == ORC_BFLOAT16);
  const double tmax = dt == ORC_DOUBLE ? 1.7976931348623157e308 : dt == ORC_HALF ? 65504.0 : dt == ORC_BFLOAT16 ? 3.3895313892515355e38 : 3.4028234663852886e38;
  PAR_FOR
  for (int64_t o = 0; o < olen; o++) {
    int64_t xb = walk(orank, oshape, oxs, o), zb = walk(orank, oshape, ozs, o);
#define XO(j) (isVector ? orc_offset(xsi, (j)) : xb + (j)*xs)
#define ZO(j) (isVector ? orc_offset(zsi, (j)) : zb + (j)*zs)
    if (dt == ORC_DOUBLE) {
      double mx = -tmax, sum = 0;
      for (int64_t j = 0; j < L; j++) { double v = ((const double *)x)[XO(j)]; if (clamp) { if (!isinf(v) && !isnan(v)) mx = v > mx ? v : mx; } else mx = v > mx ? v : mx; }
      if (clamp && mx == -tmax) mx = 0;
      for (int64_t j = 0; j < L; j++) {
        double v = ((const double *)x)[XO(j)];
        double rr;
        if (clamp) { if (isinf(v) || isnan(v)) v = (v > 0 || isnan(v)) ? 88.0 + mx : -88.0 + mx; double d = v - mx; d = d > 88.0 ? 88.0 : d; d = d < -88.0 ? -88.0 : d; rr = exp(d); }
        else rr = exp(v - mx);
        ((double *)z)[ZO(j)] = rr; sum += rr;
      }
      if (clamp) sum = sum > (double)1e-6f ? sum : (double)1e-6f;
      for (int64_t j = 0; j < L; j++) ((double *)z)[ZO(j)] /= sum;
    } else {
      /* r is carried in float (tmp) unless literal_half asks for the storage-type roundings */
      float *tmp = (float *)malloc(sizeof(float) * (size_t)L);
      float mx = (float)-tmax, sum = 0;
      for (int64_t j = 0; j < L; j++) {
        float v = ldf(x, dt, XO(j));
        if (clamp) { if (!isinf(v) && !isnan(v)) mx = v > mx ? v : mx; } else mx = v > mx ? v : mx;
      }
      if (clamp && mx == (float)-tmax) mx = 0;
      for (int64_t j = 0; j < L; j++) {
        float v = ldf(x, dt, XO(j)), d;
        if (clamp) {
          if (isinf(v) || isnan(v)) v = (v > 0 || isnan(v)) ? 88.0f + mx : -88.0f + mx;
          if (lit) v = rnd(v, dt);
          d = v - mx;
          if (lit) d = rnd(d, dt);
          d = d > 88.0f ? 88.0f : d;
          d = d < -88.0f ? -88.0f : d;
        } else {
          d = v - mx;
          if (lit) d = rnd(d, dt);
        }
        float rr = expf(d);
        if (lit) { rr = rnd(rr, dt); sum = rnd(sum + rr, dt); } else sum += rr;
        tmp[j] = rr;
      }
      if (clamp) { float eps = lit ? rnd(1e-6f, dt) : 1e-6f; sum = sum > eps ? sum : eps; }
      for (int64_t j = 0; j < L; j++) st(z, dt, ZO(j), tmp[j] / sum);
      free(tmp);
    }
#undef XO
#undef ZO
  }
  return 0;
}

/* ---------------------------------------------------------------------------------------------
 * layer_norm                                  ops/declarable/generic/nn/layer_norm.cpp:35-79
 *   = standardize (generic/transforms/standardize.cpp:34-78) * gain (+ bias, helpers/cpu/addBias.cpp)
 * mean = Mean(x, axes) (float sequential sum / n), var = population variance by Welford updates in
 * double (loops/summarystatsreduce.h:60-95,184-220) cast to the array type, stdev = sqrt(var + 1e-5),
 * y = (x - mean) / stdev * gain + bias.  gain/bias run along dim 1 (channelsFirst) or the last dim.
 * For half types every intermediate is evaluated in float and rounded once at the end (see header).
 * ------------------------------------------------------------------------------------------- */
int orc_layer_norm(const void *x, const int64_t *xsi, const void *gain, const int64_t *gsi, const void *bias,
                   const int64_t *bsi, void *z, const int64_t *zsi, const int64_t *axes, int naxes, int channelsFirst) {
  int r = si_rank(xsi), dt = orc_dtype(xsi);
  if (dt != orc_dtype(zsi) || !dt_is_float(dt)) return 2;
  if (naxes < 1) return 3;
  RedPlan p;
  if (red_plan(xsi, axes, naxes, &p)) return 3;
  int dimC = channelsFirst ? 1 : r - 1;
  if (dimC >= r) return 3;
  int64_t C = si_shape(xsi)[dimC];
  if (orc_length(gsi) != C || (bias && orc_length(bsi) != C)) return 3;
  int gdt = orc_dtype(gsi), bdt = bias ? orc_dtype(bsi) : 0;
  /* z strides for the same split */
  int red[ORC_MAX_RANK] = {0};
  for (int i = 0; i < naxes; i++) red[axes[i] < 0 ? axes[i] + r : axes[i]] = 1;
  int64_t zo_stride[ORC_MAX_RANK], zi_stride[ORC_MAX_RANK]; int a = 0, b = 0;
  /* channel coordinate of an (outer, inner) pair: track which split dimC belongs to */
  int cInInner = red[dimC], cPos = 0;
  for (int i = 0; i < r; i++) {
    if (red[i]) { if (i == dimC) cPos = b; zi_stride[b++] = si_stride(zsi)[i]; }
    else { if (i == dimC) cPos = a; zo_stride[a++] = si_stride(zsi)[i]; }
  }
  PAR_FOR
  for (int64_t o = 0; o < p.olen; o++) {
    int64_t xb = walk(p.orank, p.oshape, p.ostride, o), zb = walk(p.orank, p.oshape, zo_stride, o);
    float sumf = 0; double sumd = 0;
    double n = 0, mean = 0, M2 = 0;
    for (int64_t j = 0; j < p.ilen; j++) {
      double v = ld(x, dt, xb + walk(p.irank, p.ishape, p.istride, j));
      sumf = (float)v + sumf; sumd += v;
      /* SummaryStatsReduce::update with a single-element right operand */
      if (n == 0) { n = 1; mean = v; M2 = 0; }
      else { double nn = n + 1, delta = v - mean; mean = mean + delta * 1.0 / nn; M2 = M2 + delta * delta * n * 1.0 / nn; n = nn; }
    }
    double var = n <= 1.0 ? 0.0 : M2 / n;
    for (int64_t j = 0; j < p.ilen; j++) {
      int64_t xo = xb + walk(p.irank, p.ishape, p.istride, j), zo = zb + walk(p.irank, p.ishape, zi_stride, j);
      /* channel index of this element */
      int64_t idx = cInInner ? j : o, c = 0;
      { const int64_t *sh = cInInner ? p.ishape : p.oshape; int rk = cInInner ? p.irank : p.orank;
        for (int i = rk - 1; i >= 0; i--) { int64_t q = idx % sh[i]; idx /= sh[i]; if (i == cPos) { c = q; break; } } }
      if (dt == ORC_DOUBLE) {
        double m = sumd / (double)p.ilen, sd = sqrt(var + 1e-5);
        double y = (((const double *)x)[xo] - m) / sd * ld(gain, gdt, c);
        if (bias) y += ld(bias, bdt, c);
        ((double *)z)[zo] = y;
      } else {
        float m = sumf / (float)p.ilen, sd = sqrtf((float)var + 1e-5f);
        float y = (ldf(x, dt, xo) - m) / sd * ldf(gain, gdt, c);
        if (bias) y += ldf(bias, bdt, c);
        st(z, dt, zo, y);
      }
    }
  }
  return 0;
}

/* ---------------------------------------------------------------------------------------------
 * matmul (aliases mMul, mmul, gemm, gemv, dot) ops/declarable/generic/blas/matmul.cpp:35-176
 *   -> helpers/impl/MmulHelper.cpp:486-614 -> helpers/cpu/MmulHelper.cpp:35-110 (usualGemm), :190-306
 * C = alpha * op(A) op(B) + beta * C over leading batch dims; IArgs [transX, transY, transZ];
 * transZ swaps the inputs and flips the flags (matmul.cpp:50-56).  1-D operands: dot, vec x mat
 * ([M] -> [1,M]) and mat x vec (helpers/impl/MmulHelper.cpp:406-452).
 * fp32/fp64 go to an external BLAS in the reference (sgemm/dgemm, summation order unspecified);
 * every other dtype runs usualGemm, which multiplies and accumulates in the output type
 * (`T3 val`, cpu/MmulHelper.cpp:92-98) -- accumulate = 0 reproduces that literally.
 * ------------------------------------------------------------------------------------------- */
int orc_matmul(const void *x, const int64_t *xsi, const void *y, const int64_t *ysi, void *z, const int64_t *zsi,
               int transX, int transY, int transZ, double alpha, double beta, int accumulate) {
  if (transZ) {
    const void *t = x; x = y; y = t;
    const int64_t *ts = xsi; xsi = ysi; ysi = ts;
    int tmp = transX; transX = !transY; transY = !tmp;
  }
  int xr = si_rank(xsi), yr = si_rank(ysi), zr = si_rank(zsi);
  int xdt = orc_dtype(xsi), ydt = orc_dtype(ysi), zdt = orc_dtype(zsi);
  if (xr < 1 || yr < 1) return 3;
  int64_t M, K, N, Ky, as_m, as_k, bs_k, bs_n, cs_m, cs_n;
  int64_t batch = 1, bshape[ORC_MAX_RANK], bxs[ORC_MAX_RANK], bys[ORC_MAX_RANK], bzs[ORC_MAX_RANK]; int br = 0;
  if (xr == 1) { M = 1; K = si_shape(xsi)[0]; as_m = 0; as_k = si_stride(xsi)[0]; }
  else {
    int mi = transX ? xr - 1 : xr - 2, ki = transX ? xr - 2 : xr - 1;
    M = si_shape(xsi)[mi]; K = si_shape(xsi)[ki]; as_m = si_stride(xsi)[mi]; as_k = si_stride(xsi)[ki];
  }
  if (yr == 1) { Ky = si_shape(ysi)[0]; N = 1; bs_k = si_stride(ysi)[0]; bs_n = 0; }
  else {
    int ki = transY ? yr - 1 : yr - 2, ni = transY ? yr - 2 : yr - 1;
    Ky = si_shape(ysi)[ki]; N = si_shape(ysi)[ni]; bs_k = si_stride(ysi)[ki]; bs_n = si_stride(ysi)[ni];
  }
  if (K != Ky) return 3;
  if (xr > 2 || yr > 2) {
    if (xr != yr || xr != zr) return 3;
    br = xr - 2;
    for (int i = 0; i < br; i++) {
      if (si_shape(xsi)[i] != si_shape(ysi)[i] || si_shape(xsi)[i] != si_shape(zsi)[i]) return 3;
      bshape[i] = si_shape(xsi)[i]; bxs[i] = si_stride(xsi)[i]; bys[i] = si_stride(ysi)[i]; bzs[i] = si_stride(zsi)[i];
      batch *= bshape[i];
    }
  }
  /* z strides */
  if (orc_length(zsi) != batch * M * N) return 3;
  if (zr >= 2 && xr >= 2 && yr >= 2) { cs_m = si_stride(zsi)[zr - 2]; cs_n = si_stride(zsi)[zr - 1]; }
  else if (xr == 1 && yr == 1) { cs_m = 0; cs_n = 0; }
  else if (xr == 1) { cs_m = 0; cs_n = zr >= 1 ? si_stride(zsi)[zr - 1] : 0; }
  else { cs_m = zr >= 1 ? si_stride(zsi)[zr - 1] : 0; cs_n = 0; }
  int64_t total = batch * M * N;
  PAR_FOR
  for (int64_t t = 0; t < total; t++) {
    int64_t bidx = t / (M * N), m = (t / N) % M, n = t % N;
    int64_t ao = walk(br, bshape, bxs, bidx) + m * as_m, bo = walk(br, bshape, bys, bidx) + n * bs_n;
    int64_t co = walk(br, bshape, bzs, bidx) + m * cs_m + n * cs_n;
    double res;
    if (accumulate == 2 || zdt == ORC_DOUBLE) {
      double acc = 0;
      for (int64_t k = 0; k < K; k++) acc += ld(x, xdt, ao + k * as_k) * ld(y, ydt, bo + k * bs_k);
      res = acc;
    } else if (accumulate == 1 || zdt == ORC_FLOAT32) {
      float acc = 0;
      for (int64_t k = 0; k < K; k++) acc += ldf(x, xdt, ao + k * as_k) * ldf(y, ydt, bo + k * bs_k);
      res = acc;
    } else {
      float acc = rnd(ldf(x, xdt, ao) * ldf(y, ydt, bo), zdt);
      for (int64_t k = 1; k < K; k++) acc = rnd(acc + rnd(ldf(x, xdt, ao + k * as_k) * ldf(y, ydt, bo + k * bs_k), zdt), zdt);
      res = acc;
    }
    if (zdt == ORC_DOUBLE) {
      ((double *)z)[co] = beta != 0.0 ? alpha * res + beta * ((double *)z)[co] : alpha * res;
    } else {
      float a = rnd((float)alpha, zdt), b = rnd((float)beta, zdt), v = (float)res;
      if (accumulate == 0 && zdt != ORC_FLOAT32) {
        float t1 = rnd(a * v, zdt);
        st(z, zdt, co, beta != 0.0 ? rnd(t1 + rnd(b * ldf(z, zdt, co), zdt), zdt) : t1);
      } else {
        st(z, zdt, co, beta != 0.0 ? a * v + b * ldf(z, zdt, co) : a * v);
      }
    }
  }
  return 0;
}

/* ---------------------------------------------------------------------------------------------
 * dot_product_attention_v2                    ops/declarable/generic/nn/dot_product_attention_v2.cpp:35-125
 *   -> helpers/impl/AttentionHelper.cpp:411-469 (doAttention), :340-352 (attentionHelper),
 *      :70-79 (lowerTriangularMask), :189-241 (applyAttentionScores)
 * inputs ordered (queries, values, keys); rank 3 [batch, T, dim].
 * logits = clip(scale * q k^T, +-1e4) (scale skipped when 0 or 1); causal mask keeps j <= i; masked
 * logits get 65504 subtracted for bf16 and -- intended semantics, see header -- 1e9 otherwise;
 * weights = softmax(logits, -1) with the clamp semantics above; out = weights * v.
 * logits/weights outputs are stored rounded to the array dtype; the softmax reads the stored logits and
 * the final product reads the stored weights, as the reference's op-by-op composition does.
 * qmask [batch, Tq] / vmask [batch, Tv] (any numeric dtype, may be NULL): see the two comments in the body.
 * ------------------------------------------------------------------------------------------- */
int orc_attention_v2(const void *q, const int64_t *qsi, const void *v, const int64_t *vsi, const void *k,
                     const int64_t *ksi, void *out, const int64_t *osi, void *weights, const int64_t *wsi,
                     void *logits, const int64_t *lsi, double scale, int causal, const void *qmask,
                     const int64_t *qmsi, const void *vmask, const int64_t *vmsi) {
  if (si_rank(qsi) != 3 || si_rank(vsi) != 3 || si_rank(ksi) != 3) return 3;
  int dt = orc_dtype(qsi);
  if (!dt_is_float(dt) || dt == ORC_DOUBLE) return 2;
  int64_t B = si_shape(qsi)[0], Tq = si_shape(qsi)[1], D = si_shape(qsi)[2], Tv = si_shape(vsi)[1], Dv = si_shape(vsi)[2];
  if (si_shape(ksi)[1] != Tv || si_shape(ksi)[2] != D) return 3;
  const int64_t *qs = si_stride(qsi), *ks = si_stride(ksi), *vs = si_stride(vsi), *os = si_stride(osi);
  float *lg = (float *)malloc(sizeof(float) * (size_t)Tv * (size_t)orc_get_threads());
  int nt = orc_get_threads();
  (void)nt;
#ifdef _OPENMP
#pragma omp parallel for schedule(static) num_threads(orc_get_threads())
#endif
  for (int64_t row = 0; row < B * Tq; row++) {
#ifdef _OPENMP
    float *L = lg + (size_t)omp_get_thread_num() * Tv;
#else
    float *L = lg;
#endif
    int64_t b = row / Tq, i = row % Tq;
    for (int64_t j = 0; j < Tv; j++) {
      float acc = 0;
      for (int64_t d = 0; d < D; d++) acc += ldf(q, dt, b * qs[0] + i * qs[1] + d * qs[2]) * ldf(k, dt, b * ks[0] + j * ks[1] + d * ks[2]);
      float l = rnd(acc, dt);
      if (scale != 0.0 && scale != 1.0) l = rnd(l * rnd((float)scale, dt), dt);
      l = l > 1e4f ? rnd(1e4f, dt) : l; l = l < -1e4f ? rnd(-1e4f, dt) : l;
      /* scoresMask = value mask (cast to BOOL, expanded at -2) AND lower-triangular mask (:175-187, :434-452);
       * where it is false the logit has the penalty subtracted once (:199-221) */
      int hidden = causal && j > i;
      if (vmask && ldf(vmask, orc_dtype(vmsi), b * si_stride(vmsi)[0] + j * si_stride(vmsi)[1]) == 0.0f) hidden = 1;
      if (hidden) l = rnd(l - (dt == ORC_BFLOAT16 ? 65504.0f : 1.0e9f), dt);
      L[j] = l;
      if (logits) st(logits, dt, b * si_stride(lsi)[0] + i * si_stride(lsi)[1] + j * si_stride(lsi)[2], l);
    }
    /* softmax, same-shape-strict branch */
    const float tmax = dt == ORC_HALF ? 65504.0f : dt == ORC_BFLOAT16 ? 3.3895313892515355e38f : 3.4028234663852886e38f;
    float mx = -tmax, sum = 0;
    for (int64_t j = 0; j < Tv; j++) if (!isinf(L[j]) && !isnan(L[j])) mx = L[j] > mx ? L[j] : mx;
    if (mx == -tmax) mx = 0;
    for (int64_t j = 0; j < Tv; j++) {
      float val = L[j];
      if (isinf(val) || isnan(val)) val = (val > 0 || isnan(val)) ? 88.0f + mx : -88.0f + mx;
      float d = val - mx; d = d > 88.0f ? 88.0f : d; d = d < -88.0f ? -88.0f : d;
      L[j] = expf(d); sum += L[j];
    }
    sum = sum > 1e-6f ? sum : 1e-6f;
    for (int64_t j = 0; j < Tv; j++) L[j] = rnd(L[j] / sum, dt);
    for (int64_t d = 0; d < Dv; d++) {
      float acc = 0;
      for (int64_t j = 0; j < Tv; j++) acc += L[j] * ldf(v, dt, b * vs[0] + j * vs[1] + d * vs[2]);
      st(out, dt, b * os[0] + i * os[1] + d * os[2], acc);
    }
    /* the query mask (cast to the arrays' type, expanded at -1) multiplies the scores array after the output has
     * been formed from it (:455-467): it shows in the weights output only */
    if (weights) {
      float qm = qmask ? rnd(ldf(qmask, orc_dtype(qmsi), b * si_stride(qmsi)[0] + i * si_stride(qmsi)[1]), dt) : 1.0f;
      for (int64_t j = 0; j < Tv; j++)
        st(weights, dt, b * si_stride(wsi)[0] + i * si_stride(wsi)[1] + j * si_stride(wsi)[2], qmask ? L[j] * qm : L[j]);
    }
  }
  free(lg);
  return 0;
}

/* z[r, c] = x[r, c] + row[c]: the bias add of the decoder harness (helpers/cpu/addBias.cpp, NHWC branch) */
int orc_add_row_vector(const void *x, const int64_t *xsi, const void *row, const int64_t *rsi, void *z,
                       const int64_t *zsi) {
  int r = si_rank(xsi), dt = orc_dtype(xsi);
  int64_t C = si_shape(xsi)[r - 1], n = orc_length(xsi);
  if (orc_length(rsi) != C) return 3;
  PAR_FOR
  for (int64_t i = 0; i < n; i++) {
    float a = ldf(x, dt, orc_offset(xsi, i)), b = ldf(row, orc_dtype(rsi), orc_offset(rsi, i % C));
    st(z, orc_dtype(zsi), orc_offset(zsi, i), a + b);
  }
  return 0;
}
