// Layer normalisation of one row held by one wave, shared by the row kernel and by the products that normalise their
// input row on the way in: the same instruction sequence in both places, hence the same bits.
#pragma once
#include "device.h"

namespace nd4jhip {

// vals: the row's elements, lane t holding elements (t + 64 i) * VEC .. + VEC - 1 of pass i; keep[i] = 0 for a pass whose
// vector lies beyond the row (such lanes hold a re-read of the last vector).  On return vals holds
// (x - mean) / sqrt(var + eps) * gain (+ bias), population variance.
template <typename T, int NV, bool HAS_BIAS, int G = 64>
__device__ __forceinline__ void ln_wave_row(typename Conv<T>::acc (&vals)[NV * RawIO<T>::N], const typename RawIO<T>::raw (&gv)[NV],
                                            const typename RawIO<T>::raw (&bv)[NV], const typename Conv<T>::acc (&keep)[NV], int L, float eps) {
  using A = typename Conv<T>::acc;
  constexpr int VEC = RawIO<T>::N;
  A sum = (A)0;
#pragma unroll
  for (int i = 0; i < NV; i++) {
    A part = (A)0;
#pragma unroll
    for (int e = 0; e < VEC; e++) part += vals[i * VEC + e];
    sum += part * keep[i];
  }
  if constexpr (G == 64) sum = wave_allreduce<SumOp>(sum); else sum = group_allreduce<SumOp, G>(sum);   // G < 64: a row per G lanes
  const A mean = sum / (A)L;
  A sq = (A)0;
#pragma unroll
  for (int i = 0; i < NV; i++) {
    A part = (A)0;
#pragma unroll
    for (int e = 0; e < VEC; e++) { const A d = vals[i * VEC + e] - mean; vals[i * VEC + e] = d; part += d * d; }
    sq += part * keep[i];
  }
  if constexpr (G == 64) sq = wave_allreduce<SumOp>(sq); else sq = group_allreduce<SumOp, G>(sq);
  const A var = L > 1 ? sq / (A)L : (A)0;
  const A rstd = (A)1 / (sizeof(A) == 8 ? (A)sqrt((double)(var + (A)eps)) : (A)sqrtf((float)(var + (A)eps)));
#pragma unroll
  for (int i = 0; i < NV; i++) {
    A g[VEC], b[VEC];
    RawIO<T>::unpack(gv[i], g);
    if (HAS_BIAS) RawIO<T>::unpack(bv[i], b);
#pragma unroll
    for (int e = 0; e < VEC; e++) {
      A y = vals[i * VEC + e] * rstd * g[e];
      if (HAS_BIAS) y += b[e];
      vals[i * VEC + e] = y;
    }
  }
}

// Attention over a key range cut into `splits` parts: each part leaves (D sums of weight x value relative to its own row
// maximum, that maximum, its sum of weights) in a record of ATTN_PART_PITCH(D) floats.  N consecutive elements, from t0 on, of
// the merged and normalised output row.  The streaming attention kernel's merge kernel and the one-row product that
// reads the row right away (and merges on its way in) both call this, so they produce the same bits.
#define ATTN_PART_PITCH(D) ((D) + 4)
template <int N, int S>
__device__ __forceinline__ void attn_merge_parts(const float* __restrict__ P, int D, int t0, float (&out)[N]) {
  const float L2E = 1.44269502162933349609375f;
  const int pitch = ATTN_PART_PITCH(D);
  // every load first (the count of parts is a compile-time constant: one trip to memory, not one per part)
  float m[S], l[S], o[S][N];
  typedef __attribute__((ext_vector_type(4))) float f32x4m;
  typedef __attribute__((ext_vector_type(2))) float f32x2m;
#pragma unroll
  for (int s = 0; s < S; s++) {
    const f32x2m ml = *reinterpret_cast<const f32x2m*>(P + s * pitch + D);   // records start on 16-byte boundaries, D is a multiple of 4
    m[s] = ml[0];
    l[s] = ml[1];
    if constexpr (N % 4 == 0) {   // (t0 is then a multiple of 4 as well: 16-byte loads)
#pragma unroll
      for (int q = 0; q < N / 4; q++) {
        const f32x4m v = *reinterpret_cast<const f32x4m*>(P + s * pitch + t0 + 4 * q);
#pragma unroll
        for (int e = 0; e < 4; e++) o[s][4 * q + e] = v[e];
      }
    } else {
#pragma unroll
      for (int e = 0; e < N; e++) o[s][e] = P[s * pitch + t0 + e];
    }
  }
  float mm = -1.0e30f;
#pragma unroll
  for (int s = 0; s < S; s++) mm = __builtin_fmaxf(mm, m[s]);
  float lt = 0.f, ot[N];
#pragma unroll
  for (int e = 0; e < N; e++) ot[e] = 0.f;
#pragma unroll
  for (int s = 0; s < S; s++) {
    const float fw = __builtin_amdgcn_exp2f((m[s] - mm) * L2E);
    lt = __builtin_fmaf(l[s], fw, lt);
#pragma unroll
    for (int e = 0; e < N; e++) ot[e] = __builtin_fmaf(o[s][e], fw, ot[e]);
  }
  const float inv = lt > 0.f ? 1.f / lt : 0.f;   // one division per row, not one per element
#pragma unroll
  for (int e = 0; e < N; e++) out[e] = ot[e] * inv;
}
// splits is 2, 4 or 8 (what attentionDecodeSplits hands out)
template <int N>
__device__ __forceinline__ void attn_merge_vec(const float* __restrict__ P, int splits, int D, int t0, float (&out)[N]) {
  if (splits == 2) attn_merge_parts<N, 2>(P, D, t0, out);
  else if (splits == 4) attn_merge_parts<N, 4>(P, D, t0, out);
  else attn_merge_parts<N, 8>(P, D, t0, out);
}

}  // namespace nd4jhip
