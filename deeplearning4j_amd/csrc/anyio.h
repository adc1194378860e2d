// Element loads and stores with the storage type chosen at run time (slow, type-agnostic kernels).
#pragma once
#include <hip/hip_runtime.h>

#include "device.h"
#include "types.h"

namespace nd4jhip {

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

}  // namespace nd4jhip
