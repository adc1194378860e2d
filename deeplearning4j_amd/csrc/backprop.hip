// Gradient kernels of the row ops: softmax_bp and standardize_bp (the core of layer_norm_bp).
//
// softmax_bp (reference: libnd4j/include/ops/declarable/generic/nn/softmax.cpp:53-95)
//   gradI = s * (gradO - sum_row(s * gradO)) with s the forward output.  The reference runs five array ops with two
//   temporaries; here one wave (rows up to 2048 elements) or one block owns a row and makes two passes over it: the
//   second pass re-reads the row from cache, so the HBM traffic is the algorithmic 3 * sizeof(T) per element.
//
// standardize_bp (reference: generic/transforms/standardize.cpp:84-154, with reduce_mean_bp and reduce_stdev_bp,
//   generic/reduce/reduceStDev.cpp:109-177)
//   per statistics group of N elements, with mu = mean(x), sd = population standard deviation (no epsilon), g = eps
//   (times the gain of the element's channel when the caller is layer_norm_bp):
//     t    = g / sd                         u = t - sum(t) / N
//     D    = sum((mu - x) * g / (sd * sd))  v = divide_no_nan(x - mu, sd * N) * D
//     out  = u + v, NaN replaced by 0
//   The order of the divisions is the reference's, so that a group of equal values (sd = 0) yields NaN -> 0 as
//   it does there.  One block per group; arithmetic in float (double for fp64 arrays).
#include "device.h"
#include "kernels.h"
#include "runtime.h"

namespace nd4jhip {

struct Row3Args {
  DevShape outerG, outerS, outerZ;
  LongType rows, rowLen, gInner, sInner, zInner;
};

// TPR threads per row: 64 (four rows per block) or 256 (one row per block)
template <typename T, int TPR>
__global__ __launch_bounds__(256) void softmax_bp_rows(Row3Args a, const T* __restrict__ g, const T* __restrict__ sm, T* __restrict__ z) {
  using A = typename Conv<T>::acc;
  constexpr int ROWS = 256 / TPR;
  __shared__ A lds[4];
  const int t = threadIdx.x % TPR;
  LongType row = (LongType)blockIdx.x * ROWS + threadIdx.x / TPR;
  const bool live = row < a.rows;
  if (!live) row = a.rows - 1;   // keep the block convergent for the reduction
  const LongType gb = walk<LongType>(a.outerG, row), sb = walk<LongType>(a.outerS, row), zb = walk<LongType>(a.outerZ, row);
  A dot = (A)0;
  for (LongType j = t; j < a.rowLen; j += TPR) dot += (A)to_float(sm[sb + j * a.sInner]) * (A)to_float(g[gb + j * a.gInner]);
  if (TPR == 64) dot = wave_allreduce<SumOp>(dot);
  else dot = block_allreduce<SumOp, 4, A>(dot, lds);
  if (!live) return;
  for (LongType j = t; j < a.rowLen; j += TPR) {
    const A s = (A)to_float(sm[sb + j * a.sInner]);
    z[zb + j * a.zInner] = Conv<T>::from(s * ((A)to_float(g[gb + j * a.gInner]) - dot));
  }
}

// many short strided rows (a non-last axis): one thread per row so that neighbouring threads touch neighbouring
// addresses
template <typename T>
__global__ __launch_bounds__(256) void softmax_bp_flat(Row3Args a, const T* __restrict__ g, const T* __restrict__ sm, T* __restrict__ z) {
  using A = typename Conv<T>::acc;
  const LongType row = (LongType)blockIdx.x * 256 + threadIdx.x;
  if (row >= a.rows) return;
  const LongType gb = walk<LongType>(a.outerG, row), sb = walk<LongType>(a.outerS, row), zb = walk<LongType>(a.outerZ, row);
  A dot = (A)0;
  for (LongType j = 0; j < a.rowLen; j++) dot += (A)to_float(sm[sb + j * a.sInner]) * (A)to_float(g[gb + j * a.gInner]);
  for (LongType j = 0; j < a.rowLen; j++) {
    const A s = (A)to_float(sm[sb + j * a.sInner]);
    z[zb + j * a.zInner] = Conv<T>::from(s * ((A)to_float(g[gb + j * a.gInner]) - dot));
  }
}

template <typename T>
static void softmaxBpTyped(hipStream_t s, const void* g, const void* sm, void* z, const RowPlan& pg, const RowPlan& ps) {
  Row3Args a;
  a.outerG = pg.outerX; a.outerS = ps.outerX; a.outerZ = pg.outerZ;
  a.rows = pg.rows; a.rowLen = pg.rowLen; a.gInner = pg.xInner; a.sInner = ps.xInner; a.zInner = pg.zInner;
  const T* gt = (const T*)g; const T* st = (const T*)sm; T* zt = (T*)z;
  if (pg.zInner != 1 && pg.rows >= 4096 && pg.rowLen <= 4096) {
    hipLaunchKernelGGL((softmax_bp_flat<T>), dim3((unsigned)((pg.rows + 255) / 256)), dim3(256), 0, s, a, gt, st, zt);
  } else if (pg.rowLen <= 2048) {
    hipLaunchKernelGGL((softmax_bp_rows<T, 64>), dim3((unsigned)((pg.rows + 3) / 4)), dim3(256), 0, s, a, gt, st, zt);
  } else {
    hipLaunchKernelGGL((softmax_bp_rows<T, 256>), dim3((unsigned)pg.rows), dim3(256), 0, s, a, gt, st, zt);
  }
}

void launchSoftmaxBp(hipStream_t s, DataType dt, const void* gradO, const void* softmaxed, void* gradI, const RowPlan& pg,
                     const RowPlan& ps) {
  if (pg.rows == 0 || pg.rowLen == 0) return;
  ND4J_REQUIRE(pg.rows < (1LL << 31), "softmax_bp: too many rows");
  ND4J_REQUIRE(pg.rows == ps.rows && pg.rowLen == ps.rowLen, "softmax_bp: the row plans of gradO and the softmax output differ");
  switch (dt) {
    case FLOAT32: softmaxBpTyped<float>(s, gradO, softmaxed, gradI, pg, ps); break;
    case DOUBLE: softmaxBpTyped<double>(s, gradO, softmaxed, gradI, pg, ps); break;
    case HALF: softmaxBpTyped<f16_t>(s, gradO, softmaxed, gradI, pg, ps); break;
    case BFLOAT16: softmaxBpTyped<bf16_t>(s, gradO, softmaxed, gradI, pg, ps); break;
    default: ND4J_THROW("softmax_bp: unsupported dtype");
  }
  HIP_CHECK(hipGetLastError());
}

// ---- standardize_bp ------------------------------------------------------------------------------------------------
struct StdBpArgs {
  DevShape outerX, innerX, outerE, innerE, outerZ, innerZ;
  LongType outerLen, innerLen;
  int channelInInner, channelPos;
};
__device__ __forceinline__ LongType coord_of(const DevShape& s, LongType idx, int pos) {
  for (int d = s.rank - 1; d >= 0; d--) {
    const LongType q = idx / s.shape[d], c = idx - q * s.shape[d];
    if (d == pos) return c;
    idx = q;
  }
  return 0;
}
template <typename A> __device__ __forceinline__ A bp_sqrt(A x);
template <> __device__ __forceinline__ float bp_sqrt<float>(float x) { return sqrtf(x); }
template <> __device__ __forceinline__ double bp_sqrt<double>(double x) { return sqrt(x); }

template <typename T>
__global__ __launch_bounds__(256) void standardize_bp_groups(StdBpArgs a, const T* __restrict__ x, const T* __restrict__ e,
                                                             const T* __restrict__ gain, T* __restrict__ z) {
  using A = typename Conv<T>::acc;
  __shared__ A lds[4];
  const LongType o = blockIdx.x;
  const LongType xb = walk<LongType>(a.outerX, o), eb = walk<LongType>(a.outerE, o), zb = walk<LongType>(a.outerZ, o);
  const A n = (A)a.innerLen;
  A sum = (A)0;
  for (LongType j = threadIdx.x; j < a.innerLen; j += 256) sum += (A)to_float(x[xb + walk<LongType>(a.innerX, j)]);
  sum = block_allreduce<SumOp, 4, A>(sum, lds);
  const A mean = sum / n;
  A sq = (A)0;
  for (LongType j = threadIdx.x; j < a.innerLen; j += 256) { const A d = (A)to_float(x[xb + walk<LongType>(a.innerX, j)]) - mean; sq += d * d; }
  sq = block_allreduce<SumOp, 4, A>(sq, lds);
  const A sd = bp_sqrt<A>(sq / n);
  const A gOuter = (gain && !a.channelInInner) ? (A)to_float(gain[coord_of(a.outerX, o, a.channelPos)]) : (A)1;
  auto grad = [&](LongType j) {
    A g = (A)to_float(e[eb + walk<LongType>(a.innerE, j)]);
    if (gain) {
      // the reference stores eps * gain in the array type before standardize_bp reads it
      const A w = a.channelInInner ? (A)to_float(gain[coord_of(a.innerX, j, a.channelPos)]) : gOuter;
      g = (A)to_float(Conv<T>::from(g * w));
    }
    return g;
  };
  A st = (A)0, dd = (A)0;
  for (LongType j = threadIdx.x; j < a.innerLen; j += 256) {
    const A g = grad(j), xv = (A)to_float(x[xb + walk<LongType>(a.innerX, j)]);
    st += g / sd;
    dd += (mean - xv) * g / (sd * sd);
  }
  st = block_allreduce<SumOp, 4, A>(st, lds);
  dd = block_allreduce<SumOp, 4, A>(dd, lds);
  const A denom = sd * n;
  for (LongType j = threadIdx.x; j < a.innerLen; j += 256) {
    const A g = grad(j), xv = (A)to_float(x[xb + walk<LongType>(a.innerX, j)]);
    const A u = g / sd - st / n;
    const A v = (denom == (A)0 ? (A)0 : (xv - mean) / denom) * dd;
    A r = u + v;
    r = r != r ? (A)0 : r;
    z[zb + walk<LongType>(a.innerZ, j)] = Conv<T>::from(r);
  }
}

void launchStandardizeBp(hipStream_t s, DataType dt, const void* x, const void* eps, const void* gain, void* z,
                         const LnGenericPlan& px, const LnGenericPlan& pe) {
  if (px.outerLen == 0 || px.innerLen == 0) return;
  ND4J_REQUIRE(px.outerLen < (1LL << 31), "standardize_bp: too many groups");
  ND4J_REQUIRE(px.outerLen == pe.outerLen && px.innerLen == pe.innerLen, "standardize_bp: the plans of the input and of eps differ");
  StdBpArgs a;
  a.outerX = px.outerX; a.innerX = px.innerX; a.outerZ = px.outerZ; a.innerZ = px.innerZ;
  a.outerE = pe.outerX; a.innerE = pe.innerX;
  a.outerLen = px.outerLen; a.innerLen = px.innerLen; a.channelInInner = px.channelInInner; a.channelPos = px.channelPos;
  dim3 g((unsigned)px.outerLen), b(256);
  switch (dt) {
    case FLOAT32: hipLaunchKernelGGL((standardize_bp_groups<float>), g, b, 0, s, a, (const float*)x, (const float*)eps, (const float*)gain, (float*)z); break;
    case DOUBLE: hipLaunchKernelGGL((standardize_bp_groups<double>), g, b, 0, s, a, (const double*)x, (const double*)eps, (const double*)gain, (double*)z); break;
    case HALF: hipLaunchKernelGGL((standardize_bp_groups<f16_t>), g, b, 0, s, a, (const f16_t*)x, (const f16_t*)eps, (const f16_t*)gain, (f16_t*)z); break;
    case BFLOAT16: hipLaunchKernelGGL((standardize_bp_groups<bf16_t>), g, b, 0, s, a, (const bf16_t*)x, (const bf16_t*)eps, (const bf16_t*)gain, (bf16_t*)z); break;
    default: ND4J_THROW("standardize_bp: unsupported dtype");
  }
  HIP_CHECK(hipGetLastError());
}

}  // namespace nd4jhip
