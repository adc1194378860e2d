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
  static __device__ __forceinline__ bf16_t from(float f) {
    unsigned u = __float_as_uint(f);
    bf16_t r;
    if ((u & 0x7fffffffu) > 0x7f800000u) { r.bits = 0x7FC0; return r; }
    u += 0x7fffu + ((u >> 16) & 1u);
    r.bits = (unsigned short)(u >> 16);
    return r;
  }
};
template <> struct Conv<f16_t> {
  using acc = float;
  static __device__ __forceinline__ f16_t from(float f) { f16_t r; r.bits = __half_as_ushort(__float2half_rn(f)); return r; }
};

// 16-byte (or narrower) vector of storage elements
template <typename T, int N> struct alignas(sizeof(T) * N) Vec { T v[N]; };

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
