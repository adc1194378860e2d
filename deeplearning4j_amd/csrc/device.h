// Device-side helpers for gfx950 (wave64): storage<->float conversion, wave reductions built on DPP
// row operations plus two cross-row shuffles, and shape walks over DevShape records.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>

#include "types.h"

namespace nd4jhip {

constexpr int WAVE = 64;

// ---- storage types ---------------------------------------------------------------------------------
struct bf16_t { unsigned short bits; };
struct f16_t { unsigned short bits; };

// bf16: round-to-nearest-even, NaN -> 0x7FC0 (same rule as the reference's bfloat16::operator=(float),
// libnd4j/include/types/bfloat16.h:186-213)
__device__ __forceinline__ float to_float(bf16_t v) { return __uint_as_float(((unsigned)v.bits) << 16); }
__device__ __forceinline__ float to_float(f16_t v) { return __half2float(__ushort_as_half(v.bits)); }
__device__ __forceinline__ float to_float(float v) { return v; }
__device__ __forceinline__ double to_float(double v) { return v; }

template <typename T> struct Conv;
template <> struct Conv<float> { using acc = float; static __device__ __forceinline__ float from(float v) { return v; } };
template <> struct Conv<double> { using acc = double; static __device__ __forceinline__ double from(double v) { return v; } };
template <> struct Conv<bf16_t> {
  using acc = float;
  // gfx950 converts in hardware (v_cvt_pk_bf16_f32, round-to-nearest-even); a NaN stays a quiet NaN but
  // its payload is the hardware's, not necessarily the reference's 0x7FC0
  static __device__ __forceinline__ bf16_t from(float f) {
    // the empty asm pins the value in a register: it keeps the compiler from folding a preceding negation
    // into the conversion's source modifier, a pattern this compiler version fails to select
    asm("" : "+v"(f));
    bf16_t r;
    r.bits = __builtin_bit_cast(unsigned short, (__bf16)f);
    return r;
  }
};
template <> struct Conv<f16_t> {
  using acc = float;
  static __device__ __forceinline__ f16_t from(float f) { f16_t r; r.bits = __half_as_ushort(__float2half_rn(f)); return r; }
};

// two floats -> one register of two storage values (first in the low half), with one packed conversion for bf16
typedef __attribute__((ext_vector_type(2))) float f32x2a;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2a;
// (by reference: the caller goes on with the registers that pass through the asm, so no copies are made for it)
template <typename T> __device__ __forceinline__ unsigned pack_pair(float& a, float& b);
template <> __device__ __forceinline__ unsigned pack_pair<bf16_t>(float& a, float& b) {
  asm("" : "+v"(a), "+v"(b));   // keeps source modifiers out of the packed conversion (see Conv<bf16_t>::from)
  const f32x2a v = {a, b};
  return __builtin_bit_cast(unsigned, __builtin_convertvector(v, bf16x2a));
}
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2a;
template <> __device__ __forceinline__ unsigned pack_pair<f16_t>(float& a, float& b) {
  const f32x2a v = {a, b};
  return __builtin_bit_cast(unsigned, __builtin_convertvector(v, f16x2a));   // one packed conversion, round to nearest even
}

// 16-byte (or narrower) vector of storage elements
template <typename T, int N> struct alignas(sizeof(T) * N) Vec { T v[N]; };

// 16-byte register images per storage type, with conversion to and from the accumulation type.  Memory
// instructions (also the non-temporal ones) work on these vector types directly.
typedef __attribute__((ext_vector_type(4))) float raw_f32x4;
typedef __attribute__((ext_vector_type(2))) double raw_f64x2;
typedef __attribute__((ext_vector_type(4))) unsigned raw_u32x4;
template <typename T> struct RawIO;
template <> struct RawIO<float> {
  using raw = raw_f32x4;
  static constexpr int N = 4;
  static __device__ __forceinline__ void unpack(raw r, float* out) {
#pragma unroll
    for (int e = 0; e < 4; e++) out[e] = r[e];
  }
  static __device__ __forceinline__ raw pack(const float* in) { raw r = {in[0], in[1], in[2], in[3]}; return r; }
};
template <> struct RawIO<double> {
  using raw = raw_f64x2;
  static constexpr int N = 2;
  static __device__ __forceinline__ void unpack(raw r, double* out) { out[0] = r[0]; out[1] = r[1]; }
  static __device__ __forceinline__ raw pack(const double* in) { raw r = {in[0], in[1]}; return r; }
};
template <> struct RawIO<bf16_t> {
  using raw = raw_u32x4;
  static constexpr int N = 8;
  static __device__ __forceinline__ void unpack(raw r, float* out) {
#pragma unroll
    for (int p = 0; p < 4; p++) {
      out[2 * p] = __uint_as_float(r[p] << 16);
      out[2 * p + 1] = __uint_as_float(r[p] & 0xffff0000u);
    }
  }
  static __device__ __forceinline__ raw pack(const float* in) {
    raw r;
#pragma unroll
    for (int p = 0; p < 4; p++) {
      float lo = in[2 * p], hi = in[2 * p + 1];
      r[p] = pack_pair<bf16_t>(lo, hi);
    }
    return r;
  }
};
template <> struct RawIO<f16_t> {
  using raw = raw_u32x4;
  static constexpr int N = 8;
  static __device__ __forceinline__ void unpack(raw r, float* out) {
#pragma unroll
    for (int p = 0; p < 4; p++) {
      out[2 * p] = __half2float(__ushort_as_half((unsigned short)(r[p] & 0xffffu)));
      out[2 * p + 1] = __half2float(__ushort_as_half((unsigned short)(r[p] >> 16)));
    }
  }
  static __device__ __forceinline__ raw pack(const float* in) {
    raw r;
#pragma unroll
    // (one conversion per value: the packed fp16 conversion does not give the same bits for every input)
    for (int p = 0; p < 4; p++) {
      const unsigned lo = Conv<f16_t>::from(in[2 * p]).bits, hi = Conv<f16_t>::from(in[2 * p + 1]).bits;
      r[p] = lo | (hi << 16);
    }
    return r;
  }
};

// a naturally aligned vector of 4, 8 or 16 bytes on its way out: through a non-temporal store when `nts` says so (the hosts ask
// for it for results of 8 MiB and more), else an ordinary one; other sizes always take the ordinary store
// (the 16-byte case is written as assembly: given both stores in one branch the compiler sinks them into a single ordinary
// store and the non-temporal hint is gone)
template <typename VT>
__device__ __forceinline__ void store_vec(VT* p, const VT& v, bool nts) {
  if constexpr (sizeof(VT) == 16) {
    if (nts) {
      const raw_u32x4 q = __builtin_bit_cast(raw_u32x4, v);
      asm volatile("global_store_dwordx4 %0, %1, off nt" ::"v"(p), "v"(q) : "memory");
      return;
    }
  }
  *p = v;
}

// a 16-byte pack of elements of T on its way out through a non-temporal store, to an address that is only element-aligned
typedef unsigned u32x4_align2 __attribute__((ext_vector_type(4), aligned(2)));
typedef unsigned u32x4_align4 __attribute__((ext_vector_type(4), aligned(4)));
template <typename T, typename P>
__device__ __forceinline__ void nt_store16_elem_aligned(T* dst, const P& pack) {
  static_assert(sizeof(P) == 16 && (sizeof(T) == 2 || sizeof(T) == 4), "16-byte packs of 2- or 4-byte elements");
  if constexpr (sizeof(T) == 2) __builtin_nontemporal_store(__builtin_bit_cast(u32x4_align2, pack), reinterpret_cast<u32x4_align2*>(dst));
  else __builtin_nontemporal_store(__builtin_bit_cast(u32x4_align4, pack), reinterpret_cast<u32x4_align4*>(dst));
}

// 12-byte vectors of a 16-bit type (six values, one global_load_dwordx3): a wave pass covers 384 values, so a row of 768
// is two full passes where 16-byte vectors leave a quarter of the load slots idle.  Rows need 4-byte alignment only.
struct alignas(4) raw_u32x3 {
  unsigned v[3];
  __device__ __forceinline__ unsigned& operator[](int i) { return v[i]; }
  __device__ __forceinline__ unsigned operator[](int i) const { return v[i]; }
};
template <typename T> struct RawIO12 {
  using raw = raw_u32x3;
  static constexpr int N = 6;
  static __device__ __forceinline__ void unpack(raw r, float* out) {
#pragma unroll
    for (int p = 0; p < 3; p++) {
      T lo, hi;
      lo.bits = (unsigned short)(r[p] & 0xffffu);
      hi.bits = (unsigned short)(r[p] >> 16);
      out[2 * p] = to_float(lo);
      out[2 * p + 1] = to_float(hi);
    }
  }
  static __device__ __forceinline__ raw pack(const float* in) {
    raw r;
#pragma unroll
    for (int p = 0; p < 3; p++) {
      float lo = in[2 * p], hi = in[2 * p + 1];
      if constexpr (sizeof(typename Conv<T>::acc) == 4 && __is_same(T, bf16_t)) r[p] = pack_pair<bf16_t>(lo, hi);
      else r[p] = (unsigned)Conv<T>::from(lo).bits | ((unsigned)Conv<T>::from(hi).bits << 16);
    }
    return r;
  }
};

// ---- fast math for the fused row/activation kernels ---------------------------------------------------
// 1/x from the hardware reciprocal (1 ulp) instead of the 11-instruction IEEE division sequence
__device__ __forceinline__ float fast_rcp(float x) { return __builtin_amdgcn_rcpf(x); }
__device__ __forceinline__ double fast_rcp(double x) { return 1.0 / x; }
// e^x through v_exp_f32 with the rounding error of x*log2(e) folded back in (about 2 ulp over the whole
// range, 6 instructions); no special handling beyond what v_exp_f32 does for overflow/underflow
__device__ __forceinline__ float fast_exp(float x) {
  const float L2E = 1.44269502162933349609375f, L2E_LO = 1.925963033500011e-08f, LN2 = 0.693147182464599609375f;
  float t = x * L2E;
  float lo = __builtin_fmaf(x, L2E, -t);
  lo = __builtin_fmaf(x, L2E_LO, lo);
  lo = __builtin_fabsf(t) == INFINITY ? 0.f : lo;   // keeps e^(+-inf) = inf / 0 instead of NaN
  float r = __builtin_amdgcn_exp2f(t);
  return __builtin_fmaf(r, lo * LN2, r);
}
__device__ __forceinline__ double fast_exp(double x) { return exp(x); }

// GELU as the legacy transform evaluates it, x * sigmoid(1.702 x) (ops.h:1010-1012), in the two forms the elementwise kernels
// use: the full-precision exponential, and for dense 16-bit arrays one v_exp_f32 of x * log2(e).  GEMM epilogues that apply
// the activation call the same functions, so a fused step reproduces the separate transform bit for bit.
__device__ __forceinline__ float gelu_full(float x) { const float u = 1.702f * x; return x * fast_rcp(1.f + fast_exp(-u)); }
__device__ __forceinline__ float gelu_low(float x) { const float u = 1.702f * x; return x * fast_rcp(1.f + __builtin_amdgcn_exp2f(u * -1.44269502162933349609375f)); }

// ---- wave reductions ---------------------------------------------------------------------------------
// Butterfly over a row of 16 lanes with DPP (quad_perm 1,0,3,2 / 2,3,0,1 / row_half_mirror / row_mirror),
// then lanes 16 and 32 apart through the cross-lane permute.  Valid for commutative, associative ops;
// every lane ends up with the wave total.
template <int CTRL>
__device__ __forceinline__ float dpp_f(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true));
}
template <int CTRL>
__device__ __forceinline__ int dpp_i(int v) { return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xf, 0xf, true); }

struct SumOp { template <typename A> static __device__ __forceinline__ A apply(A a, A b) { return a + b; } };
struct MaxOp { template <typename A> static __device__ __forceinline__ A apply(A a, A b) { return a > b ? a : b; } };
struct MinOp { template <typename A> static __device__ __forceinline__ A apply(A a, A b) { return a < b ? a : b; } };
struct ProdOp { template <typename A> static __device__ __forceinline__ A apply(A a, A b) { return a * b; } };

template <typename Op>
__device__ __forceinline__ float wave_allreduce(float v) {
  v = Op::apply(v, dpp_f<0xB1>(v));   // quad_perm [1,0,3,2]
  v = Op::apply(v, dpp_f<0x4E>(v));   // quad_perm [2,3,0,1]
  v = Op::apply(v, dpp_f<0x141>(v));  // row_half_mirror
  v = Op::apply(v, dpp_f<0x140>(v));  // row_mirror
  v = Op::apply(v, __shfl_xor(v, 16, WAVE));
  v = Op::apply(v, __shfl_xor(v, 32, WAVE));
  return v;
}
// the same over aligned groups of G = 8, 16, 32 or 64 neighbouring lanes (several short rows per wave): the first levels of
// the butterfly above, each of which stays inside such a group
template <typename Op, int G>
__device__ __forceinline__ float group_allreduce(float v) {
  static_assert(G == 8 || G == 16 || G == 32 || G == 64, "group size");
  v = Op::apply(v, dpp_f<0xB1>(v));
  v = Op::apply(v, dpp_f<0x4E>(v));
  v = Op::apply(v, dpp_f<0x141>(v));
  if (G >= 16) v = Op::apply(v, dpp_f<0x140>(v));
  if (G >= 32) v = Op::apply(v, __shfl_xor(v, 16, WAVE));
  if (G >= 64) v = Op::apply(v, __shfl_xor(v, 32, WAVE));
  return v;
}
template <typename Op, int G>
__device__ __forceinline__ double group_allreduce(double v) {
#pragma unroll
  for (int m = 1; m < G; m <<= 1) v = Op::apply(v, __shfl_xor(v, m, WAVE));
  return v;
}
template <typename Op>
__device__ __forceinline__ double wave_allreduce(double v) {
#pragma unroll
  for (int m = 1; m < WAVE; m <<= 1) v = Op::apply(v, __shfl_xor(v, m, WAVE));
  return v;
}

// Block-wide all-reduce for blocks of NW waves: wave totals through LDS, then every wave folds them.
template <typename Op, int NW, typename A>
__device__ __forceinline__ A block_allreduce(A v, A* lds /* NW entries */) {
  v = wave_allreduce<Op>(v);
  if (NW == 1) return v;
  const int lane = threadIdx.x & (WAVE - 1), w = threadIdx.x / WAVE;
  __syncthreads();  // protect lds from a previous use
  if (lane == 0) lds[w] = v;
  __syncthreads();
  A r = lds[0];
#pragma unroll
  for (int i = 1; i < NW; i++) r = Op::apply(r, lds[i]);
  return r;
}

// ---- shape walks ---------------------------------------------------------------------------------
// row-major decomposition of a linear index over `s.shape`, dotted with the strides
template <typename I>
__device__ __forceinline__ LongType walk(const DevShape& s, I idx) {
  LongType off = 0;
#pragma unroll 1
  for (int d = s.rank - 1; d > 0; d--) {
    I dim = (I)s.shape[d];
    I q = idx / dim;
    off += (LongType)(idx - q * dim) * s.stride[d];
    idx = q;
  }
  if (s.rank > 0) off += (LongType)idx * s.stride[0];
  return off;
}
// same decomposition applied to two stride sets at once (input and output views of equal shape)
template <typename I>
__device__ __forceinline__ void walk2(const DevShape& a, const DevShape& b, I idx, LongType& oa, LongType& ob) {
  oa = 0; ob = 0;
#pragma unroll 1
  for (int d = a.rank - 1; d > 0; d--) {
    I dim = (I)a.shape[d];
    I q = idx / dim;
    LongType c = (LongType)(idx - q * dim);
    oa += c * a.stride[d];
    ob += c * b.stride[d];
    idx = q;
  }
  if (a.rank > 0) { oa += (LongType)idx * a.stride[0]; ob += (LongType)idx * b.stride[0]; }
}

}  // namespace nd4jhip
