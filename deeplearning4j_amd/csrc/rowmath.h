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

}  // namespace nd4jhip
