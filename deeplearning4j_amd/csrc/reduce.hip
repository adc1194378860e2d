// Reductions along dimensions and full reductions (value and index flavours).
//
// Layout: the host splits x's dims into `outer` (kept, one output each) and `inner` (reduced).
//   coop kernel   - TPR (64 or 256) threads share one output; the inner run is read with 16-byte loads
//                   when it is unit-stride, otherwise element-wise through the inner strides.  Long inner
//                   runs with few outputs are cut into `splits` segments whose partials go through the
//                   launch context's reduction scratch and a small second kernel (deterministic order).
//   flat kernel   - one thread per output walking the inner dims; used when there are many outputs and
//                   the inner run is strided, so that neighbouring threads read neighbouring addresses.
// All of these are HBM-bound: algorithmic bytes = sizeof(T) per input element + one output per row.
//
// Value semantics follow the reference's reduce functors (libnd4j/include/ops/ops.h:2363-2378,1170-1298):
// accumulate in float for fp16/bf16/fp32 and in double for fp64, post-process (mean: / n, norm2: sqrt).
// The reference accumulates each output sequentially; a tree changes the rounding order only.
// Index semantics (ops/op_macros_index_reduce.h:33-69): strict comparison from {start, 0}, so the first
// extreme wins, NaN is never selected and an all -inf row gives 0.  Here: NaN is mapped to the start
// value on load and ties resolve to the lowest index, which yields the same integer.
#include "anyio.h"
#include <cstring>
#include <mutex>
#include <string>

#include "device.h"
#include "kernels.h"
#include "runtime.h"

namespace nd4jhip {

enum PreKind { PRE_ID = 0, PRE_ABS = 1, PRE_SQ = 2, PRE_XLOGX = 3, PRE_XLOG2X = 4 };
enum PostKind { POST_ID = 0, POST_DIV_N = 1, POST_SQRT = 2, POST_NEG = 3, POST_LOG_NEG = 4 };

template <typename Op, typename A> struct Identity;
template <typename A> struct Identity<SumOp, A> { static __device__ __forceinline__ A v() { return (A)0; } };
template <typename A> struct Identity<ProdOp, A> { static __device__ __forceinline__ A v() { return (A)1; } };
template <typename A> struct Identity<MaxOp, A> { static __device__ __forceinline__ A v() { return -(A)INFINITY; } };
template <typename A> struct Identity<MinOp, A> { static __device__ __forceinline__ A v() { return (A)INFINITY; } };

template <int PRE, typename A>
__device__ __forceinline__ A pre(A x) {
  if (PRE == PRE_ABS) return x < 0 ? -x : x;
  if (PRE == PRE_SQ) return x * x;
  if (PRE == PRE_XLOGX) return x * (sizeof(A) == 8 ? (A)log((double)x) : (A)logf((float)x));      // ops.h:2147-2153
  if (PRE == PRE_XLOG2X) return x * (sizeof(A) == 8 ? (A)log2((double)x) : (A)log2f((float)x));   // ops.h:1956-1963
  return x;
}
template <typename A>
__device__ __forceinline__ A post(A s, int kind, LongType n) {
  if (kind == POST_DIV_N) return s / (A)n;
  if (kind == POST_SQRT) return sizeof(A) == 8 ? (A)sqrt((double)s) : (A)sqrtf((float)s);
  if (kind == POST_NEG) return -s;
  if (kind == POST_LOG_NEG) return sizeof(A) == 8 ? (A)log((double)-s) : (A)logf((float)-s);      // ops.h:1966-1973
  return s;
}

struct CoopArgs {
  DevShape outer, inner, zOuter;
  LongType outerLen, innerLen;
  LongType segLen;   // elements of the inner run handled by one block (== innerLen when splits == 1)
  int splits;
  int zLinear;
  int postKind;
};

// ---- value reduce, cooperative -------------------------------------------------------------------------
template <typename Op, int PRE, typename T, int TPR>
__global__ __launch_bounds__(256) void reduce_coop(CoopArgs a, const T* __restrict__ x, T* __restrict__ z,
                                                   typename Conv<T>::acc* __restrict__ partials, int vectorOk) {
  using A = typename Conv<T>::acc;
  constexpr int V = 16 / sizeof(T);
  constexpr int ROWS = 256 / TPR;
  __shared__ A lds[4];
  const int t = threadIdx.x % TPR;
  const LongType unit = (LongType)blockIdx.x * ROWS + threadIdx.x / TPR;  // (row, split) pair
  const LongType row = unit / a.splits;
  const int split = (int)(unit - row * a.splits);
  A acc = Identity<Op, A>::v();
  const bool live = row < a.outerLen;
  if (live) {
    const LongType base = walk<LongType>(a.outer, row);
    const LongType j0 = (LongType)split * a.segLen;
    LongType j1 = j0 + a.segLen;
    if (j1 > a.innerLen) j1 = a.innerLen;
    if (a.inner.rank == 1 && a.inner.stride[0] == 1) {
      const T* p = x + base;
      LongType j = j0;
      if (vectorOk) {
        using VT = Vec<T, V>;
        // vectorOk 2: the run starts anywhere (rows of an odd length): the elements up to the first 16-byte boundary are
        // read one by one, as the tail is
        LongType f0 = j0;
        if (vectorOk == 2) {
          f0 = j0 + (LongType)(((16 - (reinterpret_cast<uintptr_t>(p + j0) & 15)) & 15) / sizeof(T));
          if (f0 > j1) f0 = j1;
          for (LongType q = j0 + t; q < f0; q += TPR) acc = Op::apply(acc, pre<PRE, A>((A)to_float(p[q])));
        }
        const LongType nv = (j1 - f0) / V;
        const VT* pv = reinterpret_cast<const VT*>(p + f0);
        LongType i = t;
        for (; i + 3 * TPR < nv; i += 4 * TPR) {
          VT v0 = pv[i], v1 = pv[i + TPR], v2 = pv[i + 2 * TPR], v3 = pv[i + 3 * TPR];
#pragma unroll
          for (int e = 0; e < V; e++) {
            acc = Op::apply(acc, pre<PRE, A>((A)to_float(v0.v[e])));
            acc = Op::apply(acc, pre<PRE, A>((A)to_float(v1.v[e])));
            acc = Op::apply(acc, pre<PRE, A>((A)to_float(v2.v[e])));
            acc = Op::apply(acc, pre<PRE, A>((A)to_float(v3.v[e])));
          }
        }
        for (; i < nv; i += TPR) {
          VT v0 = pv[i];
#pragma unroll
          for (int e = 0; e < V; e++) acc = Op::apply(acc, pre<PRE, A>((A)to_float(v0.v[e])));
        }
        j = f0 + nv * V;
      }
      for (LongType q = j + t; q < j1; q += TPR) acc = Op::apply(acc, pre<PRE, A>((A)to_float(p[q])));
    } else if (a.inner.rank == 1) {
      const LongType st = a.inner.stride[0];
      for (LongType q = j0 + t; q < j1; q += TPR) acc = Op::apply(acc, pre<PRE, A>((A)to_float(x[base + q * st])));
    } else {
      for (LongType q = j0 + t; q < j1; q += TPR)
        acc = Op::apply(acc, pre<PRE, A>((A)to_float(x[base + walk<LongType>(a.inner, q)])));
    }
  }
  if (TPR == 64) acc = wave_allreduce<Op>(acc);
  else if (TPR < 64) acc = group_allreduce<Op, TPR < 64 ? TPR : 8>(acc);   // short rows: 8, 16 or 32 lanes each
  else acc = block_allreduce<Op, 4, A>(acc, lds);
  if (live && t == 0) {
    if (a.splits == 1) {
      const LongType zo = a.zLinear ? row : walk<LongType>(a.zOuter, row);
      z[zo] = Conv<T>::from(post<A>(acc, a.postKind, a.innerLen));
    } else {
      partials[unit] = acc;
    }
  }
}

template <typename Op, typename T>
__global__ __launch_bounds__(256) void reduce_finish(CoopArgs a, const typename Conv<T>::acc* __restrict__ partials,
                                                     T* __restrict__ z) {
  using A = typename Conv<T>::acc;
  const LongType row = (LongType)blockIdx.x * 256 + threadIdx.x;
  if (row >= a.outerLen) return;
  A acc = Identity<Op, A>::v();
  for (int s = 0; s < a.splits; s++) acc = Op::apply(acc, partials[row * a.splits + s]);
  const LongType zo = a.zLinear ? row : walk<LongType>(a.zOuter, row);
  z[zo] = Conv<T>::from(post<A>(acc, a.postKind, a.innerLen));
}

// few outputs, many partials each (a whole array reduced to one element: 1024 partials): a block per output, its threads
// over the partials, so that the partials cost one trip to memory and not a chain of loads in a single thread
template <typename Op, typename T>
__global__ __launch_bounds__(256) void reduce_finish_wide(CoopArgs a, const typename Conv<T>::acc* __restrict__ partials, T* __restrict__ z) {
  using A = typename Conv<T>::acc;
  __shared__ A lds[4];
  const LongType row = blockIdx.x;
  A acc = Identity<Op, A>::v();
  for (int s = threadIdx.x; s < a.splits; s += 256) acc = Op::apply(acc, partials[row * a.splits + s]);
  acc = block_allreduce<Op, 4, A>(acc, lds);
  if (threadIdx.x != 0) return;
  const LongType zo = a.zLinear ? row : walk<LongType>(a.zOuter, row);
  z[zo] = Conv<T>::from(post<A>(acc, a.postKind, a.innerLen));
}

// ---- value reduce, one thread per output -----------------------------------------------------------------
template <typename Op, int PRE, typename T>
__global__ __launch_bounds__(256) void reduce_flat(CoopArgs a, const T* __restrict__ x, T* __restrict__ z) {
  using A = typename Conv<T>::acc;
  const LongType row = (LongType)blockIdx.x * 256 + threadIdx.x;
  if (row >= a.outerLen) return;
  const LongType base = walk<LongType>(a.outer, row);
  A acc = Identity<Op, A>::v();
  if (a.inner.rank == 1) {
    const LongType st = a.inner.stride[0];
    for (LongType q = 0; q < a.innerLen; q++) acc = Op::apply(acc, pre<PRE, A>((A)to_float(x[base + q * st])));
  } else {
    for (LongType q = 0; q < a.innerLen; q++)
      acc = Op::apply(acc, pre<PRE, A>((A)to_float(x[base + walk<LongType>(a.inner, q)])));
  }
  const LongType zo = a.zLinear ? row : walk<LongType>(a.zOuter, row);
  z[zo] = Conv<T>::from(post<A>(acc, a.postKind, a.innerLen));
}

// ---- planning shared by value and index flavours -----------------------------------------------------------
struct LaunchShape {
  int tpr;
  int splits;
  LongType segLen;
  bool flat;
  int vectorOk;
  int peelOk;   // unit-stride runs whose starts are not 16-byte aligned: vector loads after a scalar head
};

static LaunchShape shapeLaunch(const ReducePlan& p, size_t elemSize, const void* x, size_t partialSize, size_t scratchBytes) {
  LaunchShape s;
  const bool unitInner = p.inner.rank == 1 && p.inner.stride[0] == 1;
  s.flat = !unitInner && p.outerLen >= 4096;
  s.tpr = p.innerLen >= 2048 ? 256 : 64;
  // short unit-stride rows: 8, 16 or 32 lanes per row (one 16-byte vector per lane), several rows per wave
  if (unitInner && p.innerLen * (LongType)elemSize <= 32 * 16) {
    const LongType lanes = (p.innerLen * (LongType)elemSize + 15) / 16;
    s.tpr = lanes <= 8 ? 8 : lanes <= 16 ? 16 : 32;
  }
  s.splits = 1;
  s.segLen = p.innerLen;
  // few outputs and a long run: cut the run so that the whole chip participates
  const LongType targetBlocks = 1024;
  const LongType rowsPerBlock = 256 / s.tpr;
  const LongType blocksNow = (p.outerLen + rowsPerBlock - 1) / rowsPerBlock;
  if (!s.flat && blocksNow < targetBlocks && p.innerLen >= 16384) {
    LongType want = targetBlocks / (blocksNow > 0 ? blocksNow : 1);
    LongType maxBySeg = p.innerLen / 8192;   // keep >= 8192 elements per segment
    if (want > maxBySeg) want = maxBySeg;
    LongType maxByScratch = (LongType)(scratchBytes / partialSize) / (p.outerLen > 0 ? p.outerLen : 1);
    if (want > maxByScratch) want = maxByScratch;
    if (want > 1) {
      s.tpr = 256;
      const LongType V = 16 / (LongType)elemSize;
      LongType seg = (p.innerLen + want - 1) / want;
      seg = (seg + 255) / 256 * 256;   // keeps segments vector-aligned
      (void)V;
      s.segLen = seg;
      s.splits = (int)((p.innerLen + seg - 1) / seg);
    }
  }
  // vector loads need 16-byte aligned row starts
  const LongType V = 16 / (LongType)elemSize;
  bool ok = unitInner && (reinterpret_cast<uintptr_t>(x) & 15) == 0;
  for (int d = 0; d < p.outer.rank && ok; d++) if (p.outer.shape[d] > 1 && p.outer.stride[d] % V != 0) ok = false;
  if (s.splits > 1 && s.segLen % V != 0) ok = false;
  s.vectorOk = ok ? 1 : 0;
  s.peelOk = unitInner ? 1 : 0;
  return s;
}

static CoopArgs makeArgs(const ReducePlan& p, const LaunchShape& s, int postKind) {
  CoopArgs a;
  a.outer = p.outer; a.inner = p.inner; a.zOuter = p.zOuter;
  a.outerLen = p.outerLen; a.innerLen = p.innerLen;
  a.segLen = s.segLen; a.splits = s.splits; a.zLinear = p.zLinear ? 1 : 0; a.postKind = postKind;
  return a;
}

// ---- value reduce, rows at a constant pitch ----------------------------------------------------------------------------
// The common shape (a dense matrix reduced along its contiguous axis) without the generality above: one block per
// row, every thread issues its NL 16-byte loads at once (lanes past the row's end re-read the last vector and
// contribute the identity), no shape walk, no loop.  Measured 20.0 us against 21.3 us for the general kernel on
// fp32 [8192, 4096], the same as a bare streaming read of the matrix.
template <typename Op, int PRE, typename T, int NL>
__global__ __launch_bounds__(256) void reduce_rows_fast(const T* __restrict__ x, T* __restrict__ z, LongType xPitch, LongType zPitch, int L, int postKind) {
  using A = typename Conv<T>::acc;
  constexpr int V = 16 / sizeof(T);
  using VT = Vec<T, V>;
  __shared__ A lds[4];
  const int t = threadIdx.x;
  const VT* p = reinterpret_cast<const VT*>(x + (LongType)blockIdx.x * xPitch);
  const int nv = L / V;
  VT v[NL];
#pragma unroll
  for (int i = 0; i < NL; i++) { const int k = t + i * 256; v[i] = p[k < nv ? k : nv - 1]; }
  A acc = Identity<Op, A>::v();
#pragma unroll
  for (int i = 0; i < NL; i++) {
    A part = Identity<Op, A>::v();
#pragma unroll
    for (int e = 0; e < V; e++) part = Op::apply(part, pre<PRE, A>((A)to_float(v[i].v[e])));
    acc = Op::apply(acc, t + i * 256 < nv ? part : Identity<Op, A>::v());
  }
  acc = block_allreduce<Op, 4, A>(acc, lds);
  if (t == 0) z[(LongType)blockIdx.x * zPitch] = Conv<T>::from(post<A>(acc, postKind, L));
}
template <typename Op, int PRE, typename T>
static bool tryReduceRowsFast(hipStream_t st, const void* x, void* z, const ReducePlan& p, const LaunchShape& s, int postKind) {
  constexpr int V = 16 / sizeof(T);
  if (s.flat || s.splits != 1 || !s.vectorOk || p.outer.rank > 1 || (!p.zLinear && p.zOuter.rank > 1)) return false;
  if (p.innerLen % V != 0 || p.innerLen < 1024 || p.innerLen > 8 * 256 * V || p.outerLen >= (1LL << 31)) return false;
  const LongType xPitch = p.outer.rank ? p.outer.stride[0] : 0;
  const LongType zPitch = p.zLinear ? 1 : (p.zOuter.rank ? p.zOuter.stride[0] : 0);
  const int nl = (int)((p.innerLen / V + 255) / 256);
  const dim3 grid((unsigned)p.outerLen);
#define RF(NL) hipLaunchKernelGGL((reduce_rows_fast<Op, PRE, T, NL>), grid, dim3(256), 0, st, (const T*)x, (T*)z, xPitch, zPitch, (int)p.innerLen, postKind)
  switch (nl) {
    case 1: RF(1); break; case 2: RF(2); break; case 3: RF(3); break; case 4: RF(4); break;
    case 5: RF(5); break; case 6: RF(6); break; case 7: RF(7); break; default: RF(8); break;
  }
#undef RF
  return true;
}

// ---- value reduce down the columns of a row-major matrix (the outputs lie next to each other in x, the reduced axis walks
// at a constant pitch: sum over dim 0 of [rows, cols], over the leading dims of [a, b, cols]) ------------------------------
// A wave reads 256 bytes of one row per load (CPL columns per lane), the four waves of a block take every fourth row of
// the block's share of the rows, eight rows in flight per wave; the waves' sums meet in LDS.  With more than one block
// down the rows (few columns) the blocks park partial sums in the layout reduce_finish reads (a column's partials next to each other: with the
// partials of one split side by side instead, so that the finishing threads read coalesced, narrow matrices measured slower --
// fp32 [393216, 64] 0.4 against 0.9 TB/s -- because each finishing thread then waits on a chain of cache misses).
template <typename Op, int PRE, typename T, int CPL>
__global__ __launch_bounds__(256) void reduce_cols(CoopArgs a, const T* __restrict__ x, T* __restrict__ z, typename Conv<T>::acc* __restrict__ partials,
                                                   LongType pitch, LongType rowsPerSplit) {
  using A = typename Conv<T>::acc;
  using Raw = Vec<T, CPL>;   // CPL columns per lane in one load of up to 16 bytes
  constexpr int UNR = CPL * sizeof(T) >= 16 ? 4 : 8;
  __shared__ A lds[4][64 * CPL];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const LongType col0 = ((LongType)blockIdx.x * 64 + lane) * CPL;
  const bool live = col0 < a.outerLen;
  const LongType r0 = (LongType)blockIdx.y * rowsPerSplit;
  LongType r1 = r0 + rowsPerSplit;
  if (r1 > a.innerLen) r1 = a.innerLen;
  A acc[CPL];
#pragma unroll
  for (int c = 0; c < CPL; c++) acc[c] = Identity<Op, A>::v();
  if (live) {
    const T* p = x + col0;
    auto take = [&](const Raw& v) {
#pragma unroll
      for (int c = 0; c < CPL; c++) acc[c] = Op::apply(acc[c], pre<PRE, A>((A)to_float(v.v[c])));
    };
    LongType r = r0 + wave;
    for (; r + 4 * (UNR - 1) < r1; r += 4 * UNR) {
      Raw v[UNR];
#pragma unroll
      for (int u = 0; u < UNR; u++) v[u] = *reinterpret_cast<const Raw*>(p + (r + 4 * u) * pitch);
#pragma unroll
      for (int u = 0; u < UNR; u++) take(v[u]);
    }
    for (; r < r1; r += 4) take(*reinterpret_cast<const Raw*>(p + r * pitch));
  }
#pragma unroll
  for (int c = 0; c < CPL; c++) lds[wave][lane * CPL + c] = acc[c];
  __syncthreads();
  if (wave != 0 || !live) return;
#pragma unroll
  for (int c = 0; c < CPL; c++) {
    A t = lds[0][lane * CPL + c];
#pragma unroll
    for (int w = 1; w < 4; w++) t = Op::apply(t, lds[w][lane * CPL + c]);
    const LongType col = col0 + c;
    if (a.splits == 1) {
      const LongType zo = a.zLinear ? col : walk<LongType>(a.zOuter, col);
      z[zo] = Conv<T>::from(post<A>(t, a.postKind, a.innerLen));
    } else {
      partials[col * a.splits + blockIdx.y] = t;   // the layout reduce_finish reads
    }
  }
}
template <typename Op, int PRE, typename T>
static bool tryReduceCols(hipStream_t st, const void* x, void* z, const ReducePlan& p, int postKind, void* scratch, size_t scratchBytes) {
  using A = typename Conv<T>::acc;
  if (p.outer.rank != 1 || p.outer.stride[0] != 1 || p.inner.rank != 1 || p.innerLen < 8 || p.outerLen < 16) return false;
  const LongType pitch = p.inner.stride[0], C = p.outerLen, R = p.innerLen;
  if (pitch < C || C >= (1LL << 31)) return false;
  // as many columns per lane as one 4-byte load holds, where every row keeps such a load aligned
  // (four bytes per lane: wider loads mean fewer blocks across the columns and more down the rows, and measured slower --
  // fp32 [24576, 1024] 2.1 against 4.0 TB/s, [3072, 8192] 4.4 against 5.3)
  int cpl = 1;
  for (int c = 4 / (int)sizeof(T); c > 1; c /= 2)
    if (C % c == 0 && pitch % c == 0 && (reinterpret_cast<uintptr_t>(x) % (c * sizeof(T))) == 0 && C >= 32 * c) { cpl = c; break; }
  const LongType gx = (C + 64 * cpl - 1) / (64 * cpl);
  // enough blocks for the chip, at least 32 rows each, partials within the scratch
  LongType splits = gx >= 1024 ? 1 : (1024 + gx - 1) / gx;
  if (splits > R / 32) splits = R / 32;
  const LongType cap = (LongType)(scratchBytes / sizeof(A)) / C;
  if (splits > cap) splits = cap;
  if (splits > 65535) splits = 65535;
  if (splits < 1) splits = 1;
  LongType rowsPerSplit = (R + splits - 1) / splits;
  rowsPerSplit = (rowsPerSplit + 3) / 4 * 4;
  splits = (R + rowsPerSplit - 1) / rowsPerSplit;
  LaunchShape s{};
  s.tpr = 256; s.splits = (int)splits; s.segLen = rowsPerSplit; s.flat = false; s.vectorOk = 0; s.peelOk = 0;
  CoopArgs a = makeArgs(p, s, postKind);
  const dim3 grid((unsigned)gx, (unsigned)splits);
#define RC(CPL) hipLaunchKernelGGL((reduce_cols<Op, PRE, T, CPL>), grid, dim3(256), 0, st, a, (const T*)x, (T*)z, (A*)scratch, pitch, rowsPerSplit)
  if (cpl == 2) { if constexpr (sizeof(T) <= 2) RC(2); }
  else RC(1);
#undef RC
  if (splits > 1) {
    if (splits >= 32 && p.outerLen <= 4096)
      hipLaunchKernelGGL((reduce_finish_wide<Op, T>), dim3((unsigned)p.outerLen), dim3(256), 0, st, a, (const A*)scratch, (T*)z);
    else
      hipLaunchKernelGGL((reduce_finish<Op, T>), dim3((unsigned)((p.outerLen + 255) / 256)), dim3(256), 0, st, a, (const A*)scratch, (T*)z);
  }
  return true;
}

template <typename Op, int PRE, typename T>
static void reduceTyped(hipStream_t st, const void* x, void* z, const ReducePlan& p, int postKind, void* scratch,
                        size_t scratchBytes) {
  using A = typename Conv<T>::acc;
  if (tryReduceCols<Op, PRE, T>(st, x, z, p, postKind, scratch, scratchBytes)) return;
  LaunchShape s = shapeLaunch(p, sizeof(T), x, sizeof(A), scratchBytes);
  CoopArgs a = makeArgs(p, s, postKind);
  if (tryReduceRowsFast<Op, PRE, T>(st, x, z, p, s, postKind)) return;
  if (s.flat) {
    hipLaunchKernelGGL((reduce_flat<Op, PRE, T>), dim3((unsigned)((p.outerLen + 255) / 256)), dim3(256), 0, st, a, (const T*)x, (T*)z);
    return;
  }
  const LongType units = p.outerLen * s.splits;
  const int vec = s.vectorOk ? 1 : (s.peelOk ? 2 : 0);
  if (s.tpr < 64) {
#define RS(G) hipLaunchKernelGGL((reduce_coop<Op, PRE, T, G>), dim3((unsigned)((units + 256 / G - 1) / (256 / G))), dim3(256), 0, st, a, (const T*)x, (T*)z, (A*)scratch, vec)
    if (s.tpr == 8) RS(8); else if (s.tpr == 16) RS(16); else RS(32);
#undef RS
  } else if (s.tpr == 64) {
    hipLaunchKernelGGL((reduce_coop<Op, PRE, T, 64>), dim3((unsigned)((units + 3) / 4)), dim3(256), 0, st, a, (const T*)x, (T*)z, (A*)scratch, vec);
  } else {
    hipLaunchKernelGGL((reduce_coop<Op, PRE, T, 256>), dim3((unsigned)units), dim3(256), 0, st, a, (const T*)x, (T*)z, (A*)scratch, vec);
  }
  if (s.splits > 1) {
    if (s.splits >= 32 && p.outerLen <= 4096)
      hipLaunchKernelGGL((reduce_finish_wide<Op, T>), dim3((unsigned)p.outerLen), dim3(256), 0, st, a, (const A*)scratch, (T*)z);
    else
      hipLaunchKernelGGL((reduce_finish<Op, T>), dim3((unsigned)((p.outerLen + 255) / 256)), dim3(256), 0, st, a, (const A*)scratch, (T*)z);
  }
}

template <typename Op, int PRE>
static void reduceDtype(hipStream_t st, DataType dt, const void* x, void* z, const ReducePlan& p, int postKind,
                        void* scratch, size_t scratchBytes) {
  switch (dt) {
    case FLOAT32: return reduceTyped<Op, PRE, float>(st, x, z, p, postKind, scratch, scratchBytes);
    case DOUBLE: return reduceTyped<Op, PRE, double>(st, x, z, p, postKind, scratch, scratchBytes);
    case HALF: return reduceTyped<Op, PRE, f16_t>(st, x, z, p, postKind, scratch, scratchBytes);
    case BFLOAT16: return reduceTyped<Op, PRE, bf16_t>(st, x, z, p, postKind, scratch, scratchBytes);
    default: ND4J_THROW("reduce: unsupported dtype");
  }
}

void launchReduce(hipStream_t st, ReduceKind k, DataType xdt, DataType zdt, const void* x, void* z, const ReducePlan& p,
                  void* scratch, size_t scratchBytes) {
  ND4J_REQUIRE(xdt == zdt, "reduce: output dtype must equal input dtype on this backend");
  ND4J_REQUIRE(p.outerLen < (1LL << 31) * 4, "reduce: too many outputs");
  if (p.outerLen == 0) return;
  if (isIntLike(xdt)) return launchIntReduce(st, (int)k, false, xdt, zdt, x, z, p, scratch, scratchBytes);
  switch (k) {
    case R_SUM: reduceDtype<SumOp, PRE_ID>(st, xdt, x, z, p, POST_ID, scratch, scratchBytes); break;
    case R_MAX: reduceDtype<MaxOp, PRE_ID>(st, xdt, x, z, p, POST_ID, scratch, scratchBytes); break;
    case R_MIN: reduceDtype<MinOp, PRE_ID>(st, xdt, x, z, p, POST_ID, scratch, scratchBytes); break;
    case R_PROD: reduceDtype<ProdOp, PRE_ID>(st, xdt, x, z, p, POST_ID, scratch, scratchBytes); break;
    case R_ASUM: reduceDtype<SumOp, PRE_ABS>(st, xdt, x, z, p, POST_ID, scratch, scratchBytes); break;
    case R_AMAX: reduceDtype<MaxOp, PRE_ABS>(st, xdt, x, z, p, POST_ID, scratch, scratchBytes); break;
    case R_AMIN: reduceDtype<MinOp, PRE_ABS>(st, xdt, x, z, p, POST_ID, scratch, scratchBytes); break;
    case R_MEAN: reduceDtype<SumOp, PRE_ID>(st, xdt, x, z, p, POST_DIV_N, scratch, scratchBytes); break;
    case R_AMEAN: reduceDtype<SumOp, PRE_ABS>(st, xdt, x, z, p, POST_DIV_N, scratch, scratchBytes); break;
    case R_NORM1: reduceDtype<SumOp, PRE_ABS>(st, xdt, x, z, p, POST_ID, scratch, scratchBytes); break;
    case R_NORM2: reduceDtype<SumOp, PRE_SQ>(st, xdt, x, z, p, POST_SQRT, scratch, scratchBytes); break;
    case R_NORMMAX: reduceDtype<MaxOp, PRE_ABS>(st, xdt, x, z, p, POST_ID, scratch, scratchBytes); break;
    case R_SQNORM: reduceDtype<SumOp, PRE_SQ>(st, xdt, x, z, p, POST_ID, scratch, scratchBytes); break;
    case R_ENTROPY: reduceDtype<SumOp, PRE_XLOGX>(st, xdt, x, z, p, POST_NEG, scratch, scratchBytes); break;
    case R_LOG_ENTROPY: reduceDtype<SumOp, PRE_XLOGX>(st, xdt, x, z, p, POST_LOG_NEG, scratch, scratchBytes); break;
    case R_SHANNON_ENTROPY: reduceDtype<SumOp, PRE_XLOG2X>(st, xdt, x, z, p, POST_NEG, scratch, scratchBytes); break;
    default: ND4J_THROW("reduce: unknown op kind");
  }
  HIP_CHECK(hipGetLastError());
}

// ---- full reduction for callers that cannot allocate ---------------------------------------------------------------
// The cross-block partials of a split full reduction normally go to the launch context's hipMalloc'ed reduction buffer.
// This variant parks them in a fixed array in the code object's own global segment, so the call needs no allocation
// at all.  Every device that loads the library holds its own copy of the array (until the process ends) at its own
// address; the host-side name is only a handle for hipGetSymbolAddress, never a device address.  Calls that overlap
// on one device share the array and race; nothing in it has to start at zero (every partial a launch reads was
// written by that launch).
static __device__ __align__(256) unsigned char scratch[NOALLOC_SCRATCH_BYTES];

namespace {
constexpr int NOALLOC_MAX_DEVICES = 64;
void* g_noAllocScratch[NOALLOC_MAX_DEVICES];   // device address of `scratch`, per device
std::mutex g_noAllocMutex;
}
void* reduceNoAllocScratch() {
  int dev = 0;
  HIP_CHECK(hipGetDevice(&dev));
  ND4J_REQUIRE(dev >= 0 && dev < NOALLOC_MAX_DEVICES, "no-alloc reduction: device ordinal out of range");
  std::lock_guard<std::mutex> g(g_noAllocMutex);
  if (g_noAllocScratch[dev] == nullptr) {
    void* p = nullptr;
    HIP_CHECK(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    ND4J_REQUIRE(p != nullptr, "no-alloc reduction: hipGetSymbolAddress returned no address");
    g_noAllocScratch[dev] = p;
  }
  return g_noAllocScratch[dev];
}
void launchReduceScalarNoAlloc(hipStream_t st, ReduceKind k, DataType dt, const void* x, LongType n, void* z) {
  ND4J_REQUIRE(n >= 1, "no-alloc reduction: length must be at least 1");
  ND4J_REQUIRE(n <= NOALLOC_MAX_ELEMENTS, "no-alloc reduction: length " + std::to_string(n) + " exceeds the maximum of " + std::to_string(NOALLOC_MAX_ELEMENTS) + " elements");
  ReducePlan p;                       // a dense vector reduced to one element
  memset(&p.outer, 0, sizeof(DevShape)); memset(&p.zOuter, 0, sizeof(DevShape)); memset(&p.inner, 0, sizeof(DevShape));
  p.inner.rank = 1; p.inner.shape[0] = n; p.inner.stride[0] = 1;
  p.outerLen = 1; p.innerLen = n; p.index32 = true; p.zLinear = true;
  launchReduce(st, k, dt, dt, x, z, p, reduceNoAllocScratch(), NOALLOC_SCRATCH_BYTES);
}

// ---- summary statistics, counts, Any / All -------------------------------------------------------------------------
// One block per (output, split): any storage type through load_any, accumulation in double as the reference's
// SummaryStatsData does (loops/summarystatsreduce.h:52-56,89-100).  A block makes its segment's (n, mean, M2) in two
// passes over the segment (the second comes out of the caches); segments merge with Chan's update
// (summarystatsreduce.h:190-211), also what the finish kernel applies across splits.
struct MiscArgs {
  DevShape outer, inner, zOuter;
  DevShape yOuter, yInner;          // second operand of the reduce3 kinds (same shapes, own strides)
  LongType outerLen, innerLen, segLen;
  int splits, kind, bias, xdt, zdt, ydt;
  double param;                     // NormP: the exponent; EqualsWithEps: the tolerance
};
__device__ __forceinline__ double block_sum(double v, double* lds) {
  const int t = threadIdx.x;
  lds[t] = v;
  __syncthreads();
  for (int w = 128; w > 0; w >>= 1) {
    if (t < w) lds[t] += lds[t + w];
    __syncthreads();
  }
  const double r = lds[0];
  __syncthreads();
  return r;
}
__device__ __forceinline__ double block_max(double v, double* lds) {
  const int t = threadIdx.x;
  lds[t] = v;
  __syncthreads();
  for (int w = 128; w > 0; w >>= 1) {
    if (t < w) lds[t] = fmax(lds[t], lds[t + w]);
    __syncthreads();
  }
  const double r = lds[0];
  __syncthreads();
  return r;
}
__device__ __forceinline__ double misc_result(const MiscArgs& a, double n, double mean, double m2, double cnt) {
  switch (a.kind) {
    case M_VARIANCE: case M_STDDEV: {
      double var = n <= 1.0 ? 0.0 : m2 / n;                       // summarystatsreduce.h:89-92
      if (a.bias) {                                               // ops.h:2157-2190: falls back when the corrected value is negative
        const double corrected = n <= 1.0 ? 0.0 : m2 / (n - 1.0);
        if (!(corrected < 0.0)) var = corrected;
      }
      return a.kind == M_STDDEV ? sqrt(var) : var;
    }
    case M_ANY: return cnt > 0.0 ? 1.0 : 0.0;                     // ops.h:1200-1206: the sum of the elements is positive
    case M_ANY_FINITE: case M_ANY_INF_OR_NAN: case M_ANY_NAN: case M_ANY_INF: case M_ANY_POSITIVE: case M_ANY_NEGATIVE: return cnt > 0.0 ? 1.0 : 0.0;
    case M_ALL: return cnt > 0.0 ? 0.0 : 1.0;                     // here cnt counts the zero elements
    // reduce3 (ops.h:117-134,483-541): mean = first sum, m2 and cnt = the two auxiliary sums
    case M3_MANHATTAN: case M3_DOT: return mean;
    case M3_EUCLIDEAN: return sqrt(mean);
    case M3_COSINE_SIMILARITY: return mean / (sqrt(m2) * sqrt(cnt));
    case M3_COSINE_DISTANCE: return 1.0 - mean / (sqrt(m2) * sqrt(cnt));
    case M3_JACCARD: return 1.0 - m2 / cnt;
    case M3_HAMMING: return mean / n;
    case M3_EQUALS_EPS: return mean > 0.0 ? 0.0 : 1.0;            // mean counts the pairs further apart than the tolerance
    case M_NORMP: return pow(cnt, 1.0 / a.param);                 // ops.h:1280-1286
    case M_REDUCE_FLOAT: {                                        // the post-processing steps of ops.h:1216-1297,1956-1975,2147-2155,2370-2377
      const int rk = (int)a.param;
      if (rk == R_MEAN || rk == R_AMEAN) return cnt / n;
      if (rk == R_NORM2) return sqrt(cnt);
      if (rk == R_ENTROPY || rk == R_SHANNON_ENTROPY) return -cnt;
      if (rk == R_LOG_ENTROPY) return log(-cnt);
      return cnt;                                                 // Norm1, NormMax, SquaredNorm
    }
    default: return cnt;
  }
}
__global__ __launch_bounds__(256) void misc_partial(MiscArgs a, const void* __restrict__ x, const void* __restrict__ y, void* __restrict__ z,
                                                    double* __restrict__ partials) {
  __shared__ double lds[256];
  const LongType unit = blockIdx.x, row = unit / a.splits;
  const int split = (int)(unit - row * a.splits);
  const LongType base = walk<LongType>(a.outer, row);
  const LongType j0 = (LongType)split * a.segLen;
  LongType j1 = j0 + a.segLen;
  if (j1 > a.innerLen) j1 = a.innerLen;
  const bool linear = a.inner.rank == 1;
  const LongType st = linear ? a.inner.stride[0] : 0;
  auto at = [&](LongType q) { return load_any(x, a.xdt, base + (linear ? q * st : walk<LongType>(a.inner, q))); };
  double n = (double)(j1 - j0), mean = 0.0, m2 = 0.0, cnt = 0.0;
  if (a.kind >= M3_MANHATTAN && a.kind < M_NORMP) {
    const LongType ybase = walk<LongType>(a.yOuter, row);
    const bool ylinear = a.yInner.rank == 1;
    const LongType yst = ylinear ? a.yInner.stride[0] : 0;
    double s0 = 0.0, s1 = 0.0, s2 = 0.0;
    for (LongType q = j0 + threadIdx.x; q < j1; q += 256) {
      const double u = at(q), v = load_any(y, a.ydt, ybase + (ylinear ? q * yst : walk<LongType>(a.yInner, q)));
      switch (a.kind) {
        case M3_MANHATTAN: s0 += fabs(u - v); break;
        case M3_EUCLIDEAN: s0 += (u - v) * (u - v); break;
        case M3_DOT: s0 += u * v; break;
        case M3_COSINE_SIMILARITY: case M3_COSINE_DISTANCE: s0 += u * v; s1 += u * u; s2 += v * v; break;
        case M3_JACCARD: s1 += u < v ? u : v; s2 += u > v ? u : v; break;
        case M3_EQUALS_EPS: s0 += fabs(u - v) <= a.param ? 0.0 : 1.0; break;   // templatemath.h:115
        default: s0 += u == v ? 0.0 : 1.0; break;   // Hamming
      }
    }
    mean = block_sum(s0, lds); m2 = block_sum(s1, lds); cnt = block_sum(s2, lds);
  } else if (a.kind == M_VARIANCE || a.kind == M_STDDEV) {
    double s = 0.0;
    for (LongType q = j0 + threadIdx.x; q < j1; q += 256) s += at(q);
    mean = n > 0 ? block_sum(s, lds) / n : 0.0;
    double d2 = 0.0;
    for (LongType q = j0 + threadIdx.x; q < j1; q += 256) { const double d = at(q) - mean; d2 += d * d; }
    m2 = block_sum(d2, lds);
  } else if (a.kind == M_REDUCE_FLOAT) {
    const int rk = (int)a.param;
    double c = 0.0;
    for (LongType q = j0 + threadIdx.x; q < j1; q += 256) {
      const double v = at(q);
      switch (rk) {
        case R_AMEAN: case R_NORM1: c += fabs(v); break;
        case R_NORMMAX: c = fmax(c, fabs(v)); break;
        case R_NORM2: case R_SQNORM: c += v * v; break;
        // the logarithm is taken in X's own type (sd_log<X, Z> casts p_log<X>'s result, templatemath.h:287-299); ShannonEntropy
        // forms the product in Z (ops.h:1956-1963)
        case R_ENTROPY: case R_LOG_ENTROPY: c += v * (a.xdt == DOUBLE ? log(v) : (double)round_as(logf((float)v), a.xdt)); break;
        case R_SHANNON_ENTROPY: {
          const double pr = v * (a.xdt == DOUBLE ? log2(v) : (double)round_as(log2f((float)v), a.xdt));
          c += a.zdt == DOUBLE ? pr : (double)round_as((float)pr, a.zdt);
          break;
        }
        default: c += v; break;   // Mean
      }
    }
    cnt = rk == R_NORMMAX ? block_max(c, lds) : block_sum(c, lds);
  } else {
    double c = 0.0;
    for (LongType q = j0 + threadIdx.x; q < j1; q += 256) {
      const double v = at(q);
      if (a.kind == M_NORMP) c += pow(fabs(v), a.param);
      else if (a.kind == M_COUNT_NONZERO) c += v == 0.0 ? 0.0 : 1.0;         // ops.h:1180-1188
      else if (a.kind == M_COUNT_ZERO || a.kind == M_ALL) c += v == 0.0 ? 1.0 : 0.0;   // ops.h:1190-1198,1208-1215
      else if (a.kind >= M_ANY_FINITE) {                               // ops.h:1139-1163, indicator of the element
        const bool nan = v != v, inf = !nan && (v - v) != (v - v);
        const bool hit = a.kind == M_ANY_FINITE ? !(nan || inf) : a.kind == M_ANY_INF_OR_NAN ? (nan || inf) : a.kind == M_ANY_NAN ? nan
                         : a.kind == M_ANY_INF ? inf : a.kind == M_ANY_POSITIVE ? v > 0.0 : v < 0.0;
        c += hit ? 1.0 : 0.0;
      }
      else c += v;                                                     // Any
    }
    cnt = block_sum(c, lds);
  }
  if (threadIdx.x != 0) return;
  if (a.splits == 1) {
    store_any(z, a.zdt, walk<LongType>(a.zOuter, row), misc_result(a, n, mean, m2, cnt));
  } else {
    double* p = partials + unit * 4;
    p[0] = n; p[1] = mean; p[2] = m2; p[3] = cnt;
  }
}
__global__ __launch_bounds__(256) void misc_finish(MiscArgs a, const double* __restrict__ partials, void* __restrict__ z) {
  const LongType row = (LongType)blockIdx.x * 256 + threadIdx.x;
  if (row >= a.outerLen) return;
  double n = 0.0, mean = 0.0, m2 = 0.0, cnt = 0.0;
  for (int s = 0; s < a.splits; s++) {
    const double* p = partials + (row * a.splits + s) * 4;
    const double nb = p[0];
    if (a.kind >= M3_MANHATTAN && a.kind < M_NORMP) { n += nb; mean += p[1]; m2 += p[2]; cnt += p[3]; continue; }
    if (nb > 0.0) {
      const double delta = p[1] - mean, tot = n + nb;
      m2 += p[2] + delta * delta * n * nb / tot;
      mean += delta * nb / tot;
      n = tot;
    }
    if (a.kind == M_REDUCE_FLOAT && (int)a.param == R_NORMMAX) cnt = fmax(cnt, p[3]);
    else cnt += p[3];
  }
  store_any(z, a.zdt, walk<LongType>(a.zOuter, row), misc_result(a, n, mean, m2, cnt));
}
void launchReduceMisc(hipStream_t st, MiscReduceKind k, DataType xdt, DataType zdt, const void* x, void* z, const ReducePlan& p,
                      bool biasCorrected, void* scratch, size_t scratchBytes, const void* y, DataType ydt, const ReducePlan* yPlan, double param) {
  if (p.outerLen == 0) return;
  MiscArgs a;
  a.param = param;
  a.outer = p.outer; a.inner = p.inner; a.zOuter = p.zOuter;
  ND4J_REQUIRE((k >= M3_MANHATTAN && k < M_NORMP) == (y != nullptr && yPlan != nullptr), "reduce: second operand mismatch");
  if (yPlan) {
    ND4J_REQUIRE(yPlan->outerLen == p.outerLen && yPlan->innerLen == p.innerLen, "reduce3: operands must have equal shapes");
    a.yOuter = yPlan->outer; a.yInner = yPlan->inner;
  } else { a.yOuter = p.outer; a.yInner = p.inner; }
  a.ydt = (int)ydt;
  a.outerLen = p.outerLen; a.innerLen = p.innerLen;
  a.kind = (int)k; a.bias = biasCorrected ? 1 : 0; a.xdt = (int)xdt; a.zdt = (int)zdt;
  // few outputs with long runs: split every run over several blocks (about 2048 blocks in flight)
  LongType splits = 1;
  if (p.outerLen < 1024 && p.innerLen > 16384) {
    splits = std::min<LongType>((2048 + p.outerLen - 1) / p.outerLen, (p.innerLen + 8191) / 8192);
    const LongType cap = (LongType)(scratchBytes / (4 * sizeof(double))) / p.outerLen;
    splits = std::max<LongType>(1, std::min(splits, cap));
  }
  a.splits = (int)splits;
  a.segLen = (p.innerLen + splits - 1) / splits;
  ND4J_REQUIRE(p.outerLen * splits < (1LL << 31), "reduce: too many outputs");
  hipLaunchKernelGGL(misc_partial, dim3((unsigned)(p.outerLen * splits)), dim3(256), 0, st, a, x, y, z, (double*)scratch);
  if (splits > 1) hipLaunchKernelGGL(misc_finish, dim3((unsigned)((p.outerLen + 255) / 256)), dim3(256), 0, st, a, (const double*)scratch, z);
  HIP_CHECK(hipGetLastError());
}

// ---- index reduce ------------------------------------------------------------------------------------------
template <typename A> struct IdxVal { A v; int i; };

// IK: 0 max, 1 min, 2 abs-max, 3 abs-min
template <int IK, typename A>
__device__ __forceinline__ A idxStart() {
  if (IK == I_MAX) return -(A)INFINITY;
  if (IK == I_AMAX) return (A)0;
  return (A)INFINITY;
}
template <int IK, typename A>
__device__ __forceinline__ A idxPre(A x) {
  if (IK == I_AMAX || IK == I_AMIN) x = x < 0 ? -x : x;
  // NaN can never win a strict comparison in the reference's scan: park it on the start value
  if (x != x) x = idxStart<IK, A>();
  return x;
}
// true if candidate (bv, bi) beats (av, ai); ties go to the lower index
template <int IK, typename A>
__device__ __forceinline__ bool idxBetter(A av, int ai, A bv, int bi) {
  if (IK == I_MAX || IK == I_AMAX) return bv > av || (bv == av && bi < ai);
  return bv < av || (bv == av && bi < ai);
}
template <int IK, typename A>
__device__ __forceinline__ void idxMerge(A& av, int& ai, A bv, int bi) {
  if (idxBetter<IK, A>(av, ai, bv, bi)) { av = bv; ai = bi; }
}
template <int IK>
__device__ __forceinline__ void wave_idx_allreduce(float& v, int& i) {
  idxMerge<IK, float>(v, i, dpp_f<0xB1>(v), dpp_i<0xB1>(i));
  idxMerge<IK, float>(v, i, dpp_f<0x4E>(v), dpp_i<0x4E>(i));
  idxMerge<IK, float>(v, i, dpp_f<0x141>(v), dpp_i<0x141>(i));
  idxMerge<IK, float>(v, i, dpp_f<0x140>(v), dpp_i<0x140>(i));
  idxMerge<IK, float>(v, i, __shfl_xor(v, 16, WAVE), __shfl_xor(i, 16, WAVE));
  idxMerge<IK, float>(v, i, __shfl_xor(v, 32, WAVE), __shfl_xor(i, 32, WAVE));
}
template <int IK, int G>
__device__ __forceinline__ void group_idx_allreduce(float& v, int& i) {   // aligned groups of G = 8, 16, 32 lanes
  idxMerge<IK, float>(v, i, dpp_f<0xB1>(v), dpp_i<0xB1>(i));
  idxMerge<IK, float>(v, i, dpp_f<0x4E>(v), dpp_i<0x4E>(i));
  idxMerge<IK, float>(v, i, dpp_f<0x141>(v), dpp_i<0x141>(i));
  if (G >= 16) idxMerge<IK, float>(v, i, dpp_f<0x140>(v), dpp_i<0x140>(i));
  if (G >= 32) idxMerge<IK, float>(v, i, __shfl_xor(v, 16, WAVE), __shfl_xor(i, 16, WAVE));
}
template <int IK, int G>
__device__ __forceinline__ void group_idx_allreduce(double& v, int& i) {
#pragma unroll
  for (int m = 1; m < G; m <<= 1) idxMerge<IK, double>(v, i, __shfl_xor(v, m, WAVE), __shfl_xor(i, m, WAVE));
}
template <int IK>
__device__ __forceinline__ void wave_idx_allreduce(double& v, int& i) {
#pragma unroll
  for (int m = 1; m < WAVE; m <<= 1) idxMerge<IK, double>(v, i, __shfl_xor(v, m, WAVE), __shfl_xor(i, m, WAVE));
}

template <typename ZT>
__device__ __forceinline__ void storeIndex(ZT* z, LongType off, int idx) { z[off] = (ZT)idx; }

template <int IK, typename T, int TPR, typename ZT, int BLOCK = 256>
__global__ __launch_bounds__(BLOCK) void index_coop(CoopArgs a, const T* __restrict__ x, ZT* __restrict__ z,
                                                    IdxVal<typename Conv<T>::acc>* __restrict__ partials, int vectorOk) {
  using A = typename Conv<T>::acc;
  constexpr int V = 16 / sizeof(T);
  constexpr int ROWS = BLOCK / TPR;
  __shared__ A ldsV[BLOCK / 64];
  __shared__ int ldsI[BLOCK / 64];
  const int t = threadIdx.x % TPR;
  const LongType unit = (LongType)blockIdx.x * ROWS + threadIdx.x / TPR;
  const LongType row = unit / a.splits;
  const int split = (int)(unit - row * a.splits);
  A bv = idxStart<IK, A>();
  int bi = 0x7fffffff;   // "no element seen": loses every tie
  const bool live = row < a.outerLen;
  if (live) {
    const LongType base = walk<LongType>(a.outer, row);
    const LongType j0 = (LongType)split * a.segLen;
    LongType j1 = j0 + a.segLen;
    if (j1 > a.innerLen) j1 = a.innerLen;
    if (a.inner.rank == 1 && a.inner.stride[0] == 1) {
      const T* p = x + base;
      LongType j = j0;
      if (vectorOk) {
        using VT = Vec<T, V>;
        // vectorOk 2: the run starts anywhere (rows of an odd length): the elements up to the first 16-byte boundary are
        // read one by one, as the tail is.  Ties go to the lower index whatever the order of the visits.
        LongType f0 = j0;
        if (vectorOk == 2) {
          f0 = j0 + (LongType)(((16 - (reinterpret_cast<uintptr_t>(p + j0) & 15)) & 15) / sizeof(T));
          if (f0 > j1) f0 = j1;
          for (LongType q = j0 + t; q < f0; q += TPR) { A c = idxPre<IK, A>((A)to_float(p[q])); if (idxBetter<IK, A>(bv, bi, c, (int)q)) { bv = c; bi = (int)q; } }
        }
        const LongType nv = (j1 - f0) / V;
        const VT* pv = reinterpret_cast<const VT*>(p + f0);
        // eight vectors per thread and trip, all asked for before the first is looked at (past the end: the last vector
        // again, not counted), so that a run of up to 8 * TPR vectors costs one trip to memory
        constexpr int UNR = 8;
        for (LongType i = t; i < nv; i += (LongType)UNR * TPR) {
          VT v[UNR];
#pragma unroll
          for (int k = 0; k < UNR; k++) { const LongType ik = i + (LongType)k * TPR; v[k] = pv[ik < nv ? ik : nv - 1]; }
#pragma unroll
          for (int k = 0; k < UNR; k++) {
            const LongType ik = i + (LongType)k * TPR;
            if (ik < nv) {
#pragma unroll
              for (int e = 0; e < V; e++) { A c = idxPre<IK, A>((A)to_float(v[k].v[e])); int ci = (int)(f0 + ik * V + e); if (idxBetter<IK, A>(bv, bi, c, ci)) { bv = c; bi = ci; } }
            }
          }
        }
        j = f0 + nv * V;
      }
      for (LongType q = j + t; q < j1; q += TPR) { A c = idxPre<IK, A>((A)to_float(p[q])); if (idxBetter<IK, A>(bv, bi, c, (int)q)) { bv = c; bi = (int)q; } }
    } else if (a.inner.rank == 1) {
      const LongType st = a.inner.stride[0];
      for (LongType q = j0 + t; q < j1; q += TPR) { A c = idxPre<IK, A>((A)to_float(x[base + q * st])); if (idxBetter<IK, A>(bv, bi, c, (int)q)) { bv = c; bi = (int)q; } }
    } else {
      for (LongType q = j0 + t; q < j1; q += TPR) { A c = idxPre<IK, A>((A)to_float(x[base + walk<LongType>(a.inner, q)])); if (idxBetter<IK, A>(bv, bi, c, (int)q)) { bv = c; bi = (int)q; } }
    }
  }
  if (TPR < 64) group_idx_allreduce<IK, TPR < 64 ? TPR : 8>(bv, bi);   // short rows: 8, 16 or 32 lanes each
  else wave_idx_allreduce<IK>(bv, bi);
  if (TPR > 64) {
    static_assert(TPR <= 64 || TPR == BLOCK, "a row takes one wave or the whole block");
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    if (lane == 0) { ldsV[w] = bv; ldsI[w] = bi; }
    __syncthreads();
    bv = ldsV[0]; bi = ldsI[0];
#pragma unroll
    for (int q = 1; q < BLOCK / 64; q++) idxMerge<IK, A>(bv, bi, ldsV[q], ldsI[q]);
  }
  if (live && t == 0) {
    if (a.splits == 1) {
      const LongType zo = a.zLinear ? row : walk<LongType>(a.zOuter, row);
      storeIndex<ZT>(z, zo, bi == 0x7fffffff ? 0 : bi);
    } else {
      partials[unit].v = bv; partials[unit].i = bi;
    }
  }
}

template <int IK, typename T, typename ZT>
__global__ __launch_bounds__(256) void index_finish(CoopArgs a, const IdxVal<typename Conv<T>::acc>* __restrict__ partials,
                                                    ZT* __restrict__ z) {
  using A = typename Conv<T>::acc;
  const LongType row = (LongType)blockIdx.x * 256 + threadIdx.x;
  if (row >= a.outerLen) return;
  A bv = idxStart<IK, A>();
  int bi = 0x7fffffff;
  for (int s = 0; s < a.splits; s++) idxMerge<IK, A>(bv, bi, partials[row * a.splits + s].v, partials[row * a.splits + s].i);
  const LongType zo = a.zLinear ? row : walk<LongType>(a.zOuter, row);
  storeIndex<ZT>(z, zo, bi == 0x7fffffff ? 0 : bi);
}

template <int IK, typename T, typename ZT>
__global__ __launch_bounds__(256) void index_flat(CoopArgs a, const T* __restrict__ x, ZT* __restrict__ z) {
  using A = typename Conv<T>::acc;
  const LongType row = (LongType)blockIdx.x * 256 + threadIdx.x;
  if (row >= a.outerLen) return;
  const LongType base = walk<LongType>(a.outer, row);
  A bv = idxStart<IK, A>();
  int bi = 0;
  for (LongType q = 0; q < a.innerLen; q++) {
    const LongType off = a.inner.rank == 1 ? q * a.inner.stride[0] : walk<LongType>(a.inner, q);
    A c = idxPre<IK, A>((A)to_float(x[base + off]));
    const bool better = (IK == I_MAX || IK == I_AMAX) ? c > bv : c < bv;
    if (better) { bv = c; bi = (int)q; }
  }
  const LongType zo = a.zLinear ? row : walk<LongType>(a.zOuter, row);
  storeIndex<ZT>(z, zo, bi);
}

// index reduce over rows at a constant pitch: the counterpart of reduce_rows_fast (all loads up front, no walk, no loop);
// a thread visits its elements in ascending index order, so the strict comparison keeps the first extreme
template <int IK, typename T, int NL, typename ZT>
__global__ __launch_bounds__(256) void index_rows_fast(const T* __restrict__ x, ZT* __restrict__ z, LongType xPitch, LongType zPitch, int L) {
  using A = typename Conv<T>::acc;
  constexpr int V = 16 / sizeof(T);
  using VT = Vec<T, V>;
  __shared__ A ldsV[4];
  __shared__ int ldsI[4];
  const int t = threadIdx.x;
  const VT* p = reinterpret_cast<const VT*>(x + (LongType)blockIdx.x * xPitch);
  const int nv = L / V;
  VT v[NL];
#pragma unroll
  for (int i = 0; i < NL; i++) { const int k = t + i * 256; v[i] = p[k < nv ? k : nv - 1]; }
  A bv = idxStart<IK, A>();
  int bi = 0x7fffffff;
#pragma unroll
  for (int i = 0; i < NL; i++) {
    const int k = t + i * 256;
    if (k < nv) {
#pragma unroll
      for (int e = 0; e < V; e++) { const A c = idxPre<IK, A>((A)to_float(v[i].v[e])); const int ci = k * V + e; if (idxBetter<IK, A>(bv, bi, c, ci)) { bv = c; bi = ci; } }
    }
  }
  wave_idx_allreduce<IK>(bv, bi);
  const int lane = t & 63, w = t >> 6;
  if (lane == 0) { ldsV[w] = bv; ldsI[w] = bi; }
  __syncthreads();
  if (t == 0) {
    bv = ldsV[0]; bi = ldsI[0];
#pragma unroll
    for (int q = 1; q < 4; q++) idxMerge<IK, A>(bv, bi, ldsV[q], ldsI[q]);
    storeIndex<ZT>(z, (LongType)blockIdx.x * zPitch, bi == 0x7fffffff ? 0 : bi);
  }
}
template <int IK, typename T, typename ZT>
static bool tryIndexRowsFast(hipStream_t st, const void* x, void* z, const ReducePlan& p, const LaunchShape& s) {
  constexpr int V = 16 / sizeof(T);
  if (s.flat || s.splits != 1 || !s.vectorOk || p.outer.rank > 1 || (!p.zLinear && p.zOuter.rank > 1)) return false;
  if (p.innerLen % V != 0 || p.innerLen < 1024 || p.innerLen > 8 * 256 * V || p.outerLen >= (1LL << 31)) return false;
  const LongType xPitch = p.outer.rank ? p.outer.stride[0] : 0;
  const LongType zPitch = p.zLinear ? 1 : (p.zOuter.rank ? p.zOuter.stride[0] : 0);
  const int nl = (int)((p.innerLen / V + 255) / 256);
  const dim3 grid((unsigned)p.outerLen);
#define XF(NL) hipLaunchKernelGGL((index_rows_fast<IK, T, NL, ZT>), grid, dim3(256), 0, st, (const T*)x, (ZT*)z, xPitch, zPitch, (int)p.innerLen)
  switch (nl) {
    case 1: XF(1); break; case 2: XF(2); break; case 3: XF(3); break; case 4: XF(4); break;
    case 5: XF(5); break; case 6: XF(6); break; case 7: XF(7); break; default: XF(8); break;
  }
#undef XF
  return true;
}

// index reduce down the columns of a row-major matrix: the counterpart of reduce_cols (a wave reads 256 bytes of one row per
// load, the four waves of a block take every fourth row of the block's share; a thread meets its rows in ascending order, so
// the strict comparison keeps the first extreme, and waves, then blocks, merge with ties going to the lower row)
template <int IK, typename T, int CPL, typename ZT>
__global__ __launch_bounds__(256) void index_cols(CoopArgs a, const T* __restrict__ x, ZT* __restrict__ z, IdxVal<typename Conv<T>::acc>* __restrict__ partials,
                                                  LongType pitch, LongType rowsPerSplit) {
  using A = typename Conv<T>::acc;
  using Raw = Vec<T, CPL>;
  constexpr int UNR = 8;
  __shared__ A ldsV[4][64 * CPL];
  __shared__ int ldsI[4][64 * CPL];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const LongType col0 = ((LongType)blockIdx.x * 64 + lane) * CPL;
  const bool live = col0 < a.outerLen;
  const LongType r0 = (LongType)blockIdx.y * rowsPerSplit;
  LongType r1 = r0 + rowsPerSplit;
  if (r1 > a.innerLen) r1 = a.innerLen;
  A bv[CPL];
  int bi[CPL];
#pragma unroll
  for (int c = 0; c < CPL; c++) { bv[c] = idxStart<IK, A>(); bi[c] = 0x7fffffff; }
  if (live) {
    const T* p = x + col0;
    auto take = [&](const Raw& v, LongType r) {
#pragma unroll
      for (int c = 0; c < CPL; c++) {
        const A cv = idxPre<IK, A>((A)to_float(v.v[c]));
        if (idxBetter<IK, A>(bv[c], bi[c], cv, (int)r)) { bv[c] = cv; bi[c] = (int)r; }
      }
    };
    LongType r = r0 + wave;
    for (; r + 4 * (UNR - 1) < r1; r += 4 * UNR) {
      Raw v[UNR];
#pragma unroll
      for (int u = 0; u < UNR; u++) v[u] = *reinterpret_cast<const Raw*>(p + (r + 4 * u) * pitch);
#pragma unroll
      for (int u = 0; u < UNR; u++) take(v[u], r + 4 * u);
    }
    for (; r < r1; r += 4) take(*reinterpret_cast<const Raw*>(p + r * pitch), r);
  }
#pragma unroll
  for (int c = 0; c < CPL; c++) { ldsV[wave][lane * CPL + c] = bv[c]; ldsI[wave][lane * CPL + c] = bi[c]; }
  __syncthreads();
  if (wave != 0 || !live) return;
#pragma unroll
  for (int c = 0; c < CPL; c++) {
    A v = ldsV[0][lane * CPL + c];
    int i = ldsI[0][lane * CPL + c];
#pragma unroll
    for (int w = 1; w < 4; w++) idxMerge<IK, A>(v, i, ldsV[w][lane * CPL + c], ldsI[w][lane * CPL + c]);
    const LongType col = col0 + c;
    if (a.splits == 1) {
      const LongType zo = a.zLinear ? col : walk<LongType>(a.zOuter, col);
      storeIndex<ZT>(z, zo, i == 0x7fffffff ? 0 : i);
    } else {
      partials[col * a.splits + blockIdx.y].v = v; partials[col * a.splits + blockIdx.y].i = i;
    }
  }
}
template <int IK, typename T, typename ZT>
static bool tryIndexCols(hipStream_t st, const void* x, void* z, const ReducePlan& p, void* scratch, size_t scratchBytes) {
  using A = typename Conv<T>::acc;
  if (p.outer.rank != 1 || p.outer.stride[0] != 1 || p.inner.rank != 1 || p.innerLen < 8 || p.outerLen < 16 || p.innerLen >= (1LL << 31)) return false;
  const LongType pitch = p.inner.stride[0], C = p.outerLen, R = p.innerLen;
  if (pitch < C || C >= (1LL << 31)) return false;
  int cpl = 1;
  if (sizeof(T) == 2 && C % 2 == 0 && pitch % 2 == 0 && (reinterpret_cast<uintptr_t>(x) & 3) == 0) cpl = 2;
  const LongType gx = (C + 64 * cpl - 1) / (64 * cpl);
  LongType splits = gx >= 1024 ? 1 : (1024 + gx - 1) / gx;
  if (splits > R / 32) splits = R / 32;
  const LongType cap = (LongType)(scratchBytes / sizeof(IdxVal<A>)) / C;
  if (splits > cap) splits = cap;
  if (splits > 65535) splits = 65535;
  if (splits < 1) splits = 1;
  LongType rowsPerSplit = (R + splits - 1) / splits;
  rowsPerSplit = (rowsPerSplit + 3) / 4 * 4;
  splits = (R + rowsPerSplit - 1) / rowsPerSplit;
  LaunchShape s{};
  s.tpr = 256; s.splits = (int)splits; s.segLen = rowsPerSplit; s.flat = false; s.vectorOk = 0; s.peelOk = 0;
  CoopArgs a = makeArgs(p, s, POST_ID);
  const dim3 grid((unsigned)gx, (unsigned)splits);
  if (cpl == 2) {
    if constexpr (sizeof(T) == 2)
      hipLaunchKernelGGL((index_cols<IK, T, 2, ZT>), grid, dim3(256), 0, st, a, (const T*)x, (ZT*)z, (IdxVal<A>*)scratch, pitch, rowsPerSplit);
  } else {
    hipLaunchKernelGGL((index_cols<IK, T, 1, ZT>), grid, dim3(256), 0, st, a, (const T*)x, (ZT*)z, (IdxVal<A>*)scratch, pitch, rowsPerSplit);
  }
  if (splits > 1)
    hipLaunchKernelGGL((index_finish<IK, T, ZT>), dim3((unsigned)((p.outerLen + 255) / 256)), dim3(256), 0, st, a, (const IdxVal<A>*)scratch, (ZT*)z);
  return true;
}

template <int IK, typename T, typename ZT>
static void indexTyped(hipStream_t st, const void* x, void* z, const ReducePlan& p, void* scratch, size_t scratchBytes) {
  using A = typename Conv<T>::acc;
  if (tryIndexCols<IK, T, ZT>(st, x, z, p, scratch, scratchBytes)) return;
  LaunchShape s = shapeLaunch(p, sizeof(T), x, sizeof(IdxVal<A>), scratchBytes);
  CoopArgs a = makeArgs(p, s, POST_ID);
  if (tryIndexRowsFast<IK, T, ZT>(st, x, z, p, s)) return;
  const int vec = s.vectorOk ? 1 : (s.peelOk ? 2 : 0);
  // a few long rows (the logits of a decode step): one block of 1024 threads per row instead of segments plus a finishing
  // launch -- at this size the second launch costs more than the narrower read (kernel time for bf16 [32, 50257]:
  // 9.6 + 2.6 us in two launches, 9.0 us in one; [1, 50257] 6.6 + 2.7 against 8.0; rows of 200003 are faster cut up)
  if (s.splits > 1 && vec && p.outerLen <= 64 && p.innerLen <= (1 << 16)) {
    LaunchShape one = s;
    one.splits = 1; one.segLen = p.innerLen; one.tpr = 1024;
    CoopArgs a1 = makeArgs(p, one, POST_ID);
    hipLaunchKernelGGL((index_coop<IK, T, 1024, ZT, 1024>), dim3((unsigned)p.outerLen), dim3(1024), 0, st, a1, (const T*)x, (ZT*)z, (IdxVal<A>*)scratch, vec);
    return;
  }
  if (s.flat) {
    hipLaunchKernelGGL((index_flat<IK, T, ZT>), dim3((unsigned)((p.outerLen + 255) / 256)), dim3(256), 0, st, a, (const T*)x, (ZT*)z);
    return;
  }
  const LongType units = p.outerLen * s.splits;
  if (s.tpr < 64) {
#define IS(G) hipLaunchKernelGGL((index_coop<IK, T, G, ZT>), dim3((unsigned)((units + 256 / G - 1) / (256 / G))), dim3(256), 0, st, a, (const T*)x, (ZT*)z, (IdxVal<A>*)scratch, vec)
    if (s.tpr == 8) IS(8); else if (s.tpr == 16) IS(16); else IS(32);
#undef IS
  } else if (s.tpr == 64)
    hipLaunchKernelGGL((index_coop<IK, T, 64, ZT>), dim3((unsigned)((units + 3) / 4)), dim3(256), 0, st, a, (const T*)x, (ZT*)z, (IdxVal<A>*)scratch, vec);
  else
    hipLaunchKernelGGL((index_coop<IK, T, 256, ZT>), dim3((unsigned)units), dim3(256), 0, st, a, (const T*)x, (ZT*)z, (IdxVal<A>*)scratch, vec);
  if (s.splits > 1)
    hipLaunchKernelGGL((index_finish<IK, T, ZT>), dim3((unsigned)((p.outerLen + 255) / 256)), dim3(256), 0, st, a, (const IdxVal<A>*)scratch, (ZT*)z);
}
template <int IK, typename ZT>
static void indexDtype(hipStream_t st, DataType dt, const void* x, void* z, const ReducePlan& p, void* scratch, size_t scratchBytes) {
  switch (dt) {
    case FLOAT32: return indexTyped<IK, float, ZT>(st, x, z, p, scratch, scratchBytes);
    case DOUBLE: return indexTyped<IK, double, ZT>(st, x, z, p, scratch, scratchBytes);
    case HALF: return indexTyped<IK, f16_t, ZT>(st, x, z, p, scratch, scratchBytes);
    case BFLOAT16: return indexTyped<IK, bf16_t, ZT>(st, x, z, p, scratch, scratchBytes);
    default: ND4J_THROW("index reduce: unsupported input dtype");
  }
}
template <int IK>
static void indexKind(hipStream_t st, DataType xdt, DataType zdt, const void* x, void* z, const ReducePlan& p, void* scratch, size_t scratchBytes) {
  if (zdt == INT64) return indexDtype<IK, LongType>(st, xdt, x, z, p, scratch, scratchBytes);
  if (zdt == INT32) return indexDtype<IK, int>(st, xdt, x, z, p, scratch, scratchBytes);
  ND4J_THROW("index reduce: output must be INT32 or INT64");
}
void launchIndexReduce(hipStream_t st, IndexKind k, DataType xdt, DataType zdt, const void* x, void* z,
                       const ReducePlan& p, void* scratch, size_t scratchBytes) {
  ND4J_REQUIRE(p.innerLen < 0x7fffffffLL, "index reduce: sub-array longer than 2^31-1 elements");
  if (p.outerLen == 0) return;
  if (isIntLike(xdt)) return launchIntReduce(st, (int)k, true, xdt, zdt, x, z, p, scratch, scratchBytes);
  switch (k) {
    case I_MAX: indexKind<I_MAX>(st, xdt, zdt, x, z, p, scratch, scratchBytes); break;
    case I_MIN: indexKind<I_MIN>(st, xdt, zdt, x, z, p, scratch, scratchBytes); break;
    case I_AMAX: indexKind<I_AMAX>(st, xdt, zdt, x, z, p, scratch, scratchBytes); break;
    case I_AMIN: indexKind<I_AMIN>(st, xdt, zdt, x, z, p, scratch, scratchBytes); break;
    default: ND4J_THROW("index reduce: unknown op kind");
  }
  HIP_CHECK(hipGetLastError());
}


// ---- top-k along the last axis -------------------------------------------------------------------------------
// generic/parity_ops/top_k.cpp:31-57 -> helpers/cpu/top_k.cpp:34-125.  One block per row, k rounds of selection:
// round j picks the largest element that comes after the previous pick in the total order "greater value first,
// lower index first", so values come out in descending order and equal values in index order; NaN sorts below
// every number.  With sorted = false the k picks are put in index order afterwards.
struct TopKArgs {
  DevShape outerX, outerV, outerI;
  LongType rows, rowLen, xInner, vInner, iInner;
  int k, sorted;
};
template <typename A> struct Pick { A v; int i; };
template <typename A>
__device__ __forceinline__ bool pickBefore(A av, int ai, A bv, int bi) { return av > bv || (av == bv && ai < bi); }
template <typename T, typename ZT>
__global__ __launch_bounds__(256) void topk_rows(TopKArgs a, const T* __restrict__ x, T* __restrict__ v, ZT* __restrict__ idx) {
  using A = typename Conv<T>::acc;
  __shared__ A wv[4];
  __shared__ int wi[4];
  extern __shared__ __attribute__((aligned(8))) unsigned char picked_raw[];   // k picks when an index sort follows
  int* pickedIdx = reinterpret_cast<int*>(picked_raw);
  const LongType row = blockIdx.x;
  const LongType xb = walk<LongType>(a.outerX, row), vb = walk<LongType>(a.outerV, row), ib = walk<LongType>(a.outerI, row);
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const A LOWEST = -(A)INFINITY;
  A pv = (A)INFINITY;
  int pi = -1;
  for (int j = 0; j < a.k; j++) {
    A bv = LOWEST;
    int bi = 0x7fffffff;
    for (LongType e = t; e < a.rowLen; e += 256) {
      A c = (A)to_float(x[xb + e * a.xInner]);
      c = c == c ? c : LOWEST;                                    // NaN below everything
      const bool after = pickBefore<A>(pv, pi, c, (int)e);       // strictly after the previous pick
      if (after && pickBefore<A>(c, (int)e, bv, bi)) { bv = c; bi = (int)e; }
    }
#pragma unroll
    for (int m = 1; m < 64; m <<= 1) {
      const A ov = __shfl_xor(bv, m, WAVE);
      const int oi = __shfl_xor(bi, m, WAVE);
      if (pickBefore<A>(ov, oi, bv, bi)) { bv = ov; bi = oi; }
    }
    __syncthreads();
    if (lane == 0) { wv[wave] = bv; wi[wave] = bi; }
    __syncthreads();
    bv = wv[0]; bi = wi[0];
#pragma unroll
    for (int w = 1; w < 4; w++) if (pickBefore<A>(wv[w], wi[w], bv, bi)) { bv = wv[w]; bi = wi[w]; }
    pv = bv; pi = bi;
    if (a.sorted) {
      if (t == 0) {
        if (v) v[vb + j * a.vInner] = x[xb + (LongType)bi * a.xInner];
        if (idx) idx[ib + j * a.iInner] = (ZT)bi;
      }
    } else if (t == 0) {
      pickedIdx[j] = bi;
    }
  }
  if (!a.sorted) {
    __syncthreads();
    if (t == 0) {
      for (int j = 1; j < a.k; j++) {           // insertion sort by index (k is small)
        const int cur = pickedIdx[j];
        int q = j - 1;
        while (q >= 0 && pickedIdx[q] > cur) { pickedIdx[q + 1] = pickedIdx[q]; q--; }
        pickedIdx[q + 1] = cur;
      }
      for (int j = 0; j < a.k; j++) {
        if (v) v[vb + j * a.vInner] = x[xb + (LongType)pickedIdx[j] * a.xInner];
        if (idx) idx[ib + j * a.iInner] = (ZT)pickedIdx[j];
      }
    }
  }
}

template <typename T>
static void topkTyped(hipStream_t st, const TopKArgs& a, DataType idt, const void* x, void* v, void* idx) {
  const size_t lds = a.sorted ? 0 : (size_t)a.k * sizeof(int);
  if (idt == INT64) hipLaunchKernelGGL((topk_rows<T, LongType>), dim3((unsigned)a.rows), dim3(256), lds, st, a, (const T*)x, (T*)v, (LongType*)idx);
  else if (idt == INT32) hipLaunchKernelGGL((topk_rows<T, int>), dim3((unsigned)a.rows), dim3(256), lds, st, a, (const T*)x, (T*)v, (int*)idx);
  else ND4J_THROW("top_k: indices must be INT32 or INT64");
}
void launchTopK(hipStream_t st, DataType xdt, DataType idt, const void* x, void* values, void* indices, const RowPlan& pv,
                const RowPlan& pi, int k, bool sorted) {
  if (pv.rows == 0 || k == 0) return;
  ND4J_REQUIRE(pv.rowLen < 0x7fffffffLL && pv.rows < 0x7fffffffLL, "top_k: array too large");
  ND4J_REQUIRE(k <= 4096, "top_k: nd4j-hip selects at most 4096 elements per row");
  TopKArgs a;
  a.outerX = pv.outerX; a.outerV = pv.outerZ; a.outerI = pi.outerZ;
  a.rows = pv.rows; a.rowLen = pv.rowLen; a.xInner = pv.xInner; a.vInner = pv.zInner; a.iInner = pi.zInner;
  a.k = k; a.sorted = sorted ? 1 : 0;
  switch (xdt) {
    case FLOAT32: topkTyped<float>(st, a, idt, x, values, indices); break;
    case DOUBLE: topkTyped<double>(st, a, idt, x, values, indices); break;
    case HALF: topkTyped<f16_t>(st, a, idt, x, values, indices); break;
    case BFLOAT16: topkTyped<bf16_t>(st, a, idt, x, values, indices); break;
    default: ND4J_THROW("top_k: nd4j-hip implements floating point inputs");
  }
  HIP_CHECK(hipGetLastError());
}

}  // namespace nd4jhip
