// Attention kernels for dot_product_attention_v2.
//
//   logits fix-up - in-place pass over dense [B, Tq, Tv] logits: optional scale, clip to +-1e4, and the
//                   causal mask penalty (reference: helpers/impl/AttentionHelper.cpp:340-352, :189-241).
#include "device.h"
#include "kernels.h"
#include "runtime.h"

namespace nd4jhip {

template <typename T>
__global__ __launch_bounds__(256) void logits_fixup(T* __restrict__ l, LongType total, LongType Tq, LongType Tv, float scale,
                                                    int applyScale, int causal, float maskValue) {
  const LongType step = (LongType)gridDim.x * 256;
  for (LongType i = (LongType)blockIdx.x * 256 + threadIdx.x; i < total; i += step) {
    const LongType j = i % Tv, r = (i / Tv) % Tq;
    // every step rounds through the storage type, as the reference's op-by-op composition does
    float v = to_float(l[i]);
    if (applyScale) v = to_float(Conv<T>::from(v * to_float(Conv<T>::from(scale))));
    v = v > 1e4f ? to_float(Conv<T>::from(1e4f)) : v;
    v = v < -1e4f ? to_float(Conv<T>::from(-1e4f)) : v;
    if (causal && j > r) v = v - maskValue;
    l[i] = Conv<T>::from(v);
  }
}

void launchAttentionLogitsFixup(hipStream_t s, DataType dt, void* logits, const AttnDesc& d) {
  const LongType total = d.B * d.Tq * d.Tv;
  if (total == 0) return;
  if (!d.applyScale && !d.causal) {
    // clip only; still needed because values beyond +-1e4 must be clamped
  }
  LongType blocks = (total + 255) / 256;
  if (blocks > 256 * 16) blocks = 256 * 16;
  dim3 g((unsigned)blocks), b(256);
  switch (dt) {
    case FLOAT32: hipLaunchKernelGGL((logits_fixup<float>), g, b, 0, s, (float*)logits, total, d.Tq, d.Tv, d.scale, (int)d.applyScale, (int)d.causal, d.maskValue); break;
    case HALF: hipLaunchKernelGGL((logits_fixup<f16_t>), g, b, 0, s, (f16_t*)logits, total, d.Tq, d.Tv, d.scale, (int)d.applyScale, (int)d.causal, d.maskValue); break;
    case BFLOAT16: hipLaunchKernelGGL((logits_fixup<bf16_t>), g, b, 0, s, (bf16_t*)logits, total, d.Tq, d.Tv, d.scale, (int)d.applyScale, (int)d.causal, d.maskValue); break;
    default: ND4J_THROW("attention: unsupported dtype");
  }
  HIP_CHECK(hipGetLastError());
}

bool attentionFusedSupported(DataType, const AttnDesc&) { return false; }
void launchAttentionFused(hipStream_t, DataType, const void*, const void*, const void*, void*, const AttnDesc&) {
  ND4J_THROW("attention: fused kernel is not available in this build");
}

}  // namespace nd4jhip
