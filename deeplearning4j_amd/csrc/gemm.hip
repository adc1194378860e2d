// GEMM kernels: C = alpha * op(A) op(B) + beta * C, batched through blockIdx.z.
//
//   gemm_simple - any float dtype, any strides: 32x32 output tile per block staged through LDS, fp32
//                 (fp64 for DOUBLE) accumulation.  Correctness path for small, odd-shaped or oddly strided
//                 problems.
// The MFMA kernels for fp16/bf16/fp32 live further down and take over whenever their alignment
// requirements hold.
#include "device.h"
#include "kernels.h"
#include "runtime.h"

namespace nd4jhip {

struct GemmArgs {
  LongType M, N, K;
  LongType aRow, aCol, bRow, bCol, cRow, cCol;
  LongType aBatch, bBatch, cBatch;
  float alpha, beta;
};

template <typename T>
__global__ __launch_bounds__(256) void gemm_simple(GemmArgs g, const T* __restrict__ A, const T* __restrict__ B, T* __restrict__ C) {
  using Acc = typename Conv<T>::acc;
  constexpr int TS = 32, KS = 16;
  __shared__ Acc sa[KS][TS + 1];
  __shared__ Acc sb[KS][TS + 1];
  const LongType bz = blockIdx.z;
  A += bz * g.aBatch; B += bz * g.bBatch; C += bz * g.cBatch;
  const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;  // each thread: 2x2 outputs
  const LongType m0 = (LongType)blockIdx.y * TS, n0 = (LongType)blockIdx.x * TS;
  Acc acc[2][2] = {{0, 0}, {0, 0}};
  for (LongType k0 = 0; k0 < g.K; k0 += KS) {
    // 512 elements per operand tile, 256 threads: two each
    for (int e = threadIdx.x; e < KS * TS; e += 256) {
      const int kk = e / TS, mm = e % TS;
      const LongType k = k0 + kk;
      sa[kk][mm] = (m0 + mm < g.M && k < g.K) ? (Acc)to_float(A[(m0 + mm) * g.aRow + k * g.aCol]) : (Acc)0;
      sb[kk][mm] = (n0 + mm < g.N && k < g.K) ? (Acc)to_float(B[k * g.bRow + (n0 + mm) * g.bCol]) : (Acc)0;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < KS; kk++) {
      Acc a0 = sa[kk][ty], a1 = sa[kk][ty + 16], b0 = sb[kk][tx], b1 = sb[kk][tx + 16];
      acc[0][0] += a0 * b0; acc[0][1] += a0 * b1; acc[1][0] += a1 * b0; acc[1][1] += a1 * b1;
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 2; i++)
#pragma unroll
    for (int j = 0; j < 2; j++) {
      const LongType m = m0 + ty + 16 * i, n = n0 + tx + 16 * j;
      if (m < g.M && n < g.N) {
        const LongType off = m * g.cRow + n * g.cCol;
        Acc v = (Acc)g.alpha * acc[i][j];
        if (g.beta != 0.f) v += (Acc)g.beta * (Acc)to_float(C[off]);
        C[off] = Conv<T>::from(v);
      }
    }
}

static GemmArgs toArgs(const GemmDesc& d) {
  GemmArgs g;
  g.M = d.M; g.N = d.N; g.K = d.K;
  g.aRow = d.aRow; g.aCol = d.aCol; g.bRow = d.bRow; g.bCol = d.bCol; g.cRow = d.cRow; g.cCol = d.cCol;
  g.aBatch = d.aBatch; g.bBatch = d.bBatch; g.cBatch = d.cBatch;
  g.alpha = d.alpha; g.beta = d.beta;
  return g;
}

template <typename T>
static void launchSimple(hipStream_t s, const void* A, const void* B, void* C, const GemmDesc& d) {
  GemmArgs g = toArgs(d);
  dim3 grid((unsigned)((d.N + 31) / 32), (unsigned)((d.M + 31) / 32), (unsigned)d.batch);
  hipLaunchKernelGGL((gemm_simple<T>), grid, dim3(256), 0, s, g, (const T*)A, (const T*)B, (T*)C);
}

void launchGemm(hipStream_t s, DataType dt, const void* A, const void* B, void* C, const GemmDesc& d) {
  if (d.M == 0 || d.N == 0 || d.batch == 0) return;
  ND4J_REQUIRE(d.batch < 65536 && (d.M + 31) / 32 < 65536, "matmul: problem too large for the fallback grid");
  switch (dt) {
    case FLOAT32: launchSimple<float>(s, A, B, C, d); break;
    case DOUBLE: launchSimple<double>(s, A, B, C, d); break;
    case HALF: launchSimple<f16_t>(s, A, B, C, d); break;
    case BFLOAT16: launchSimple<bf16_t>(s, A, B, C, d); break;
    default: ND4J_THROW("matmul: unsupported dtype");
  }
  HIP_CHECK(hipGetLastError());
}

}  // namespace nd4jhip
