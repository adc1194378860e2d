// GEMM kernels: C = alpha * op(A) op(B) + beta * C, batched through blockIdx.z.
//
//   gemm_mfma16  fp16 / bf16 inputs, fp32 accumulation on the matrix cores (v_mfma_f32_32x32x16_{f16,bf16}).
//                Block tile BM x BN x 64, double-buffered through LDS.  Both operand tiles sit in LDS as
//                [k/8][row][8 k-values] (16 bytes per (k-group,row), one padding slot per k-group), which is
//                exactly what one MFMA lane consumes, so fragment reads are conflict-free ds_read_b128.
//                An operand whose K axis is contiguous in memory is copied 16 bytes at a time; an operand
//                whose M/N axis is contiguous (plain row-major B, column-major A) is loaded as 8x8 blocks and
//                transposed in registers with byte permutes on the way into LDS -- no transposed copy of
//                the matrix is ever materialised.  Workgroup ids are re-mapped so that the 32 CUs of one XCD
//                work on neighbouring tiles and share operand panels in that XCD's L2.
//                Bound: MFMA (2*M*N*K flop against the dtype's dense peak).
//   gemm_mfma32  fp32 on v_mfma_f32_32x32x2f32, tile BM x BN x 16, LDS layout [k][row].
//   gemv_*       M == 1 or N == 1: HBM-bound streaming of the matrix operand.
//   gemm_simple  any float dtype, any strides (also fp64): 32x32 tile per block through LDS.  Correctness
//                path for small, odd-shaped or oddly strided problems.
#include <cstdarg>
#include <cstdio>
#include <cstdlib>

#include <mutex>

#include "device.h"
#include <type_traits>

#include "kernels.h"
#include "mfma_tile.h"
#include "rowmath.h"
#include "runtime.h"

namespace nd4jhip {

struct GemmArgs {
  LongType M, N, K;
  LongType aRow, aCol, bRow, bCol, cRow, cCol;
  LongType aBatch, bBatch, cBatch;
  LongType batchInner;                 // > 0: batch index = outer * batchInner + inner, outer strides below
  LongType aBatch2, bBatch2, cBatch2;
  float alpha, beta;
  // split-K (16-bit MFMA kernel): blockIdx.y owns ktPerSplit K-tiles and parks its partial tile in `partial`;
  // splitk_finish adds the partials up in split order and writes C
  int splits;
  LongType ktPerSplit;
  float* partial;
  const void* bias;   // optional [N] row added to every output row (xw_plus_b), same type as C
  int hasEpi;
  GemmEpilogue epi;   // extra outputs derived from the stored C (kernels that call epilogueExtras)
  // layer-norm prologue over the rows of A (gemm_skinny32 with its LN flag only)
  const void* lnGain;
  const void* lnBias;
  void* lnOut;
  LongType lnOutRow;
  float lnEps;
};
typedef __attribute__((ext_vector_type(4))) float f32x4v;

// Name of the kernel the calling thread's most recent matmul launched ("family<tile,flags>"), so that a test can assert
// which instantiation its shape reached.
static thread_local char g_lastGemmKernel[96] = "";
__attribute__((format(printf, 1, 2))) static void noteKernel(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_lastGemmKernel, sizeof(g_lastGemmKernel), fmt, ap);
  va_end(ap);
}
const char* lastGemmKernel() { return g_lastGemmKernel; }
template <typename T> static const char* tname() { return std::is_same<T, bf16_t>::value ? "bf16" : std::is_same<T, f16_t>::value ? "f16" : std::is_same<T, float>::value ? "f32" : "f64"; }

// operand offsets of batch entry bz (one or two batch levels)
__device__ __forceinline__ void batchOffsets(const GemmArgs& g, LongType bz, LongType& oa, LongType& ob, LongType& oc) {
  if (g.batchInner > 0) {
    const LongType hi = bz / g.batchInner, lo = bz - hi * g.batchInner;
    oa = hi * g.aBatch2 + lo * g.aBatch; ob = hi * g.bBatch2 + lo * g.bBatch; oc = hi * g.cBatch2 + lo * g.cBatch;
  } else {
    oa = bz * g.aBatch; ob = bz * g.bBatch; oc = bz * g.cBatch;
  }
}

// the extra outputs of a fused step, from the value just stored to C[row][col]
template <typename T>
__device__ __forceinline__ void epilogueExtras(int hasEpi, const GemmEpilogue& epi, LongType row, LongType col, T yv) {
  if (!hasEpi) return;
  const float y = to_float(yv);
  if (epi.act) static_cast<T*>(epi.actOut)[row * epi.actRow + col] = Conv<T>::from(epi.act == 1 ? gelu_low(y) : gelu_full(y));
#pragma unroll
  for (int i = 0; i < 2; i++)
    if (i < epi.nCopy && col >= epi.copy[i].c0 && col < epi.copy[i].c1)
      static_cast<T*>(epi.copy[i].dst)[row * epi.copy[i].dstRow + col - epi.copy[i].c0] = yv;
  if (epi.resOut)
    static_cast<T*>(epi.resOut)[row * epi.resOutRow + col] = Conv<T>::from(to_float(static_cast<const T*>(epi.resIn)[row * epi.resInRow + col]) + y);
}
template <typename T>
__device__ __forceinline__ void epilogueExtras(const GemmArgs& g, LongType row, LongType col, T yv) { epilogueExtras<T>(g.hasEpi, g.epi, row, col, yv); }
// The same for four consecutive columns of one row held by one lane (col a multiple of 4, 16-bit T): 8-byte loads and
// stores wherever the target's rows and column range allow them, the element path otherwise.  Same values either way.
template <typename T>
__device__ __forceinline__ void epilogueExtras4(const GemmArgs& g, LongType row, LongType col, const float (&v)[4]) {
  if (!g.hasEpi) return;
  const GemmEpilogue& epi = g.epi;
  T yv[4];
#pragma unroll
  for (int e = 0; e < 4; e++) yv[e] = Conv<T>::from(v[e]);
  auto pack4 = [](const T (&q)[4]) { u32x2 o; o[0] = (unsigned)q[0].bits | ((unsigned)q[1].bits << 16); o[1] = (unsigned)q[2].bits | ((unsigned)q[3].bits << 16); return o; };
  auto ok8 = [](const void* p, LongType pitch) { return (reinterpret_cast<uintptr_t>(p) & 7) == 0 && pitch % 4 == 0; };
  if (epi.act) {
    T a[4];
#pragma unroll
    for (int e = 0; e < 4; e++) { const float y = to_float(yv[e]); a[e] = Conv<T>::from(epi.act == 1 ? gelu_low(y) : gelu_full(y)); }
    T* dst = static_cast<T*>(epi.actOut) + row * epi.actRow + col;
    if (ok8(epi.actOut, epi.actRow)) *reinterpret_cast<u32x2*>(dst) = pack4(a);
    else {
#pragma unroll
      for (int e = 0; e < 4; e++) dst[e] = a[e];
    }
  }
#pragma unroll
  for (int i = 0; i < 2; i++) {
    if (i >= epi.nCopy) break;
    const auto& c = epi.copy[i];
    if (col + 4 <= c.c0 || col >= c.c1) continue;
    T* dst = static_cast<T*>(c.dst) + row * c.dstRow + (col - c.c0);
    if (col >= c.c0 && col + 4 <= c.c1 && ok8(c.dst, c.dstRow) && c.c0 % 4 == 0) *reinterpret_cast<u32x2*>(dst) = pack4(yv);
    else {
#pragma unroll
      for (int e = 0; e < 4; e++) if (col + e >= c.c0 && col + e < c.c1) dst[e] = yv[e];
    }
  }
  if (epi.resOut) {
    const T* in = static_cast<const T*>(epi.resIn) + row * epi.resInRow + col;
    T* out = static_cast<T*>(epi.resOut) + row * epi.resOutRow + col;
    T r[4];
    if (ok8(epi.resIn, epi.resInRow)) {
      const u32x2 w = *reinterpret_cast<const u32x2*>(in);
      r[0].bits = (unsigned short)(w[0] & 0xffffu); r[1].bits = (unsigned short)(w[0] >> 16);
      r[2].bits = (unsigned short)(w[1] & 0xffffu); r[3].bits = (unsigned short)(w[1] >> 16);
    } else {
#pragma unroll
      for (int e = 0; e < 4; e++) r[e] = in[e];
    }
#pragma unroll
    for (int e = 0; e < 4; e++) r[e] = Conv<T>::from(to_float(r[e]) + to_float(yv[e]));
    if (ok8(epi.resOut, epi.resOutRow)) *reinterpret_cast<u32x2*>(out) = pack4(r);
    else {
#pragma unroll
      for (int e = 0; e < 4; e++) out[e] = r[e];
    }
  }
}

// ---- fallback --------------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void gemm_simple(GemmArgs g, const T* __restrict__ A, const T* __restrict__ B, T* __restrict__ C) {
  using Acc = typename Conv<T>::acc;
  constexpr int TS = 32, KS = 16;
  __shared__ Acc sa[KS][TS + 1];
  __shared__ Acc sb[KS][TS + 1];
  const LongType bz = blockIdx.z;
  { LongType oa, ob, oc; batchOffsets(g, bz, oa, ob, oc); A += oa; B += ob; C += oc; }
  const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;  // each thread: 2x2 outputs
  const LongType m0 = (LongType)blockIdx.y * TS, n0 = (LongType)blockIdx.x * TS;
  Acc acc[2][2] = {{0, 0}, {0, 0}};
  for (LongType k0 = 0; k0 < g.K; k0 += KS) {
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
        if (g.bias) v += (Acc)to_float(static_cast<const T*>(g.bias)[n]);
        C[off] = Conv<T>::from(v);
      }
    }
}

// Integer arrays (INT32 / INT64): the reference's plain loop in the array's own type (helpers/cpu/MmulHelper.cpp:35-110:
// val += A * B in T3, then alphaZ * val (+ betaZ * C) with alpha and beta cast to T3).  Sums and products in 64-bit
// integers narrowed on the store are the same values (two's complement wrap-around).  One thread per element of C.
template <typename T>
__global__ __launch_bounds__(256) void gemm_int(GemmArgs g, const T* __restrict__ A, const T* __restrict__ B, T* __restrict__ C, LongType alphaZ, LongType betaZ,
                                                int betaPresent) {
  const LongType bz = blockIdx.z;
  { LongType oa, ob, oc; batchOffsets(g, bz, oa, ob, oc); A += oa; B += ob; C += oc; }
  const LongType idx = (LongType)blockIdx.x * 256 + threadIdx.x;
  if (idx >= g.M * g.N) return;
  const LongType m = idx / g.N, n = idx - m * g.N;
  const T* a = A + m * g.aRow;
  const T* b = B + n * g.bCol;
  unsigned long long acc = 0;
  for (LongType k = 0; k < g.K; k++) acc += (unsigned long long)(LongType)a[k * g.aCol] * (unsigned long long)(LongType)b[k * g.bRow];
  const LongType off = m * g.cRow + n * g.cCol;
  unsigned long long v = (unsigned long long)alphaZ * acc;
  if (betaPresent) v += (unsigned long long)betaZ * (unsigned long long)(LongType)C[off];
  C[off] = (T)v;
}

// ---- tile scheduling ---------------------------------------------------------------------------------------------
// Hardware hands consecutive workgroup ids to the 8 XCDs round-robin.  Give every XCD a contiguous range of
// tiles instead, and walk that range in groups of GROUP_M tile-rows so that concurrently running workgroups
// of one XCD share A and B panels in its L2.
__device__ __forceinline__ void tileOf(unsigned bid, unsigned nb, unsigned tilesM, unsigned tilesN, unsigned& tm, unsigned& tn) {
  constexpr unsigned XCDS = 8, GROUP_M = 4;
  unsigned tile = bid;
  if (nb >= XCDS * 4) {
    const unsigned xcd = bid % XCDS, q = bid / XCDS;
    const unsigned per = nb / XCDS, rem = nb % XCDS;
    tile = xcd * per + (xcd < rem ? xcd : rem) + q;
  }
  const unsigned perGroup = GROUP_M * tilesN;
  const unsigned group = tile / perGroup, inGroup = tile % perGroup;
  const unsigned firstM = group * GROUP_M;
  const unsigned gsz = tilesM - firstM < GROUP_M ? tilesM - firstM : GROUP_M;
  tm = firstM + inGroup % gsz;
  tn = inGroup / gsz;
}

// Stores a wave's TM x TN accumulator tiles of 32 x 32: lane owns column (lane % 32); register r of a tile is row
// 8*(r/4) + 4*(lane/32) + r%4.  Whether C is read back (beta) and whether a bias row is added is decided once, outside
// the element loops: left inside, the compiler keeps two branches and a wait per element (5 us of a 4096^3 launch).
template <typename T, int TM, int TN, bool BOUNDS, bool HAS_BETA, bool HAS_BIAS>
__device__ __forceinline__ void storeAccTilesImpl(const GemmArgs& g, T* __restrict__ C, const f32x16 (&acc)[TM][TN], LongType rowBase, LongType colBase,
                                                  int lane) {
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int j = 0; j < TN; j++) {
      const LongType col = colBase + j * 32 + (lane & 31);
      if (BOUNDS && col >= g.N) continue;
      const float bj = HAS_BIAS ? to_float(static_cast<const T*>(g.bias)[col]) : 0.f;
      const LongType row0 = rowBase + i * 32 + 4 * (lane >> 5);
      T* p = C + row0 * g.cRow + col * g.cCol;
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const int dr = 8 * (r / 4) + (r & 3);
        if (BOUNDS && row0 + dr >= g.M) continue;
        T* q = p + (LongType)dr * g.cRow;
        float v = g.alpha * acc[i][j][r];
        if (HAS_BETA) v += g.beta * to_float(*q);
        if (HAS_BIAS) v += bj;
        *q = Conv<T>::from(v);
      }
    }
}
template <typename T, int TM, int TN, bool BOUNDS>
__device__ __forceinline__ void storeAccTiles(const GemmArgs& g, T* __restrict__ C, const f32x16 (&acc)[TM][TN], LongType rowBase, LongType colBase, int lane) {
  if (g.beta != 0.f) {
    if (g.bias) storeAccTilesImpl<T, TM, TN, BOUNDS, true, true>(g, C, acc, rowBase, colBase, lane);
    else storeAccTilesImpl<T, TM, TN, BOUNDS, true, false>(g, C, acc, rowBase, colBase, lane);
  } else if (g.bias) {
    storeAccTilesImpl<T, TM, TN, BOUNDS, false, true>(g, C, acc, rowBase, colBase, lane);
  } else {
    storeAccTilesImpl<T, TM, TN, BOUNDS, false, false>(g, C, acc, rowBase, colBase, lane);
  }
}

// split-K: park a block's partial tile (split blockIdx.y) for splitk_finish.  Layout of one partial tile:
// [q-group (i, j, r / 4)][thread][4 floats] -- 16-byte accesses, coalesced over the block.  A q-group holds 4 consecutive
// rows of one column; groups whose rows all lie beyond M are skipped.  rowBase / colBase: the wave's corner of the tile.
template <int TM, int TN, int NT>
__device__ __forceinline__ void storePartialTile(const GemmArgs& g, const f32x16 (&acc)[TM][TN], LongType tileLinear, LongType rowBase, LongType colBase,
                                                 int t, int lane) {
  constexpr int Q = TM * TN * 4;
  f32x4v* const mine = reinterpret_cast<f32x4v*>(g.partial) + (tileLinear * g.splits + blockIdx.y) * (LongType)(Q * NT);
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int j = 0; j < TN; j++)
#pragma unroll
      for (int q = 0; q < 4; q++) {
        const int idx = (i * TN + j) * 4 + q;
        if (rowBase + i * 32 + 8 * q + 4 * (lane >> 5) < g.M && colBase + j * 32 + (lane & 31) < g.N) {
          const f32x4v v = {acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]};
          mine[idx * NT + t] = v;
        }
      }
}

// ---- 16-bit MFMA kernel ----------------------------------------------------------------------------------------------
template <typename T, int BM, int BN, int WM, int WN, bool A_KC, bool B_KC>
__global__ __launch_bounds__(WM * WN * 64) void gemm_mfma16(GemmArgs g, const T* __restrict__ A, const T* __restrict__ B, T* __restrict__ C,
                                                             unsigned tilesM, unsigned tilesN) {
  constexpr int BK = 64, NT = WM * WN * 64;
  constexpr int WTM = BM / WM, WTN = BN / WN, TM = WTM / 32, TN = WTN / 32;
  using LayA = TileLayout<BM, A_KC>;
  using LayB = TileLayout<BN, B_KC>;
  constexpr int SLOTS_A = LayA::SLOTS, SLOTS_B = LayB::SLOTS, STAGE = SLOTS_A + SLOTS_B;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  u32x4* smem = reinterpret_cast<u32x4*>(smem_raw);

  unsigned tm, tn;
  tileOf(blockIdx.x, gridDim.x, tilesM, tilesN, tm, tn);
  const LongType m0 = (LongType)tm * BM, n0 = (LongType)tn * BN;
  const LongType bz = blockIdx.z;
  { LongType oa, ob, oc; batchOffsets(g, bz, oa, ob, oc); A += oa; B += ob; C += oc; }
  const LongType lda = A_KC ? g.aRow : g.aCol, ldb = B_KC ? g.bCol : g.bRow;

  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int wm = wave / WN, wn = wave % WN;

  f32x16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int j = 0; j < TN; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

  TileLoader<BM, NT, A_KC> la;
  TileLoader<BN, NT, B_KC> lb;
  LongType kt0 = 0, KT = (g.K + BK - 1) / BK;
  if (g.splits > 1) {
    kt0 = (LongType)blockIdx.y * g.ktPerSplit;
    KT = kt0 + g.ktPerSplit < KT ? kt0 + g.ktPerSplit : KT;
  }

  la.load(A, lda, m0, g.M, kt0 * BK, g.K, t);
  lb.load(B, ldb, n0, g.N, kt0 * BK, g.K, t);
  la.store(smem, t);
  lb.store(smem + SLOTS_A, t);
  __syncthreads();

  for (LongType kt = kt0; kt < KT; kt++) {
    const int cur = (int)((kt - kt0) & 1);
    if (kt + 1 < KT) {
      la.load(A, lda, m0, g.M, (kt + 1) * BK, g.K, t);
      lb.load(B, ldb, n0, g.N, (kt + 1) * BK, g.K, t);
    }
    const u32x4* sA = smem + cur * STAGE;
    const u32x4* sB = sA + SLOTS_A;
#pragma unroll
    for (int ks = 0; ks < BK / 16; ks++) {
      const int kg = ks * 2 + (lane >> 5);
      u32x4 fa[TM], fb[TN];
#pragma unroll
      for (int i = 0; i < TM; i++) fa[i] = sA[LayA::slot(kg, wm * WTM + i * 32 + (lane & 31))];
#pragma unroll
      for (int j = 0; j < TN; j++) fb[j] = sB[LayB::slot(kg, wn * WTN + j * 32 + (lane & 31))];
#pragma unroll
      for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++) acc[i][j] = Mfma16<T>::mma(fa[i], fb[j], acc[i][j]);
    }
    if (kt + 1 < KT) {
      u32x4* dst = smem + (cur ^ 1) * STAGE;
      la.store(dst, t);
      lb.store(dst + SLOTS_A, t);
    }
    __syncthreads();
  }

  // lane owns column (lane % 32); register r of a 32x32 tile is row 8*(r/4) + 4*(lane/32) + r%4
  if (g.splits > 1) {
    storePartialTile<TM, TN, NT>(g, acc, (bz * tilesM + tm) * tilesN + tn, m0 + wm * WTM, n0 + wn * WTN, t, lane);
    return;
  }
  storeAccTiles<T, TM, TN, true>(g, C, acc, m0 + wm * WTM, n0 + wn * WTN, lane);
}

// Second half of a split-K product: one block per (output tile, q-group), same thread -> element mapping as
// gemm_mfma16; adds the partial tiles in split order (deterministic), applies alpha / beta and writes C.
template <typename T, int BM, int BN, int WM, int WN>
__global__ __launch_bounds__(WM * WN * 64) void splitk_finish(GemmArgs g, T* __restrict__ C, unsigned tilesM, unsigned tilesN) {
  constexpr int NT = WM * WN * 64;
  constexpr int WTM = BM / WM, WTN = BN / WN, TM = WTM / 32, TN = WTN / 32, Q = TM * TN * 4;
  const unsigned tm = blockIdx.x / tilesN, tn = blockIdx.x % tilesN;
  const LongType m0 = (LongType)tm * BM, n0 = (LongType)tn * BN, bz = blockIdx.z;
  { LongType oa, ob, oc; batchOffsets(g, bz, oa, ob, oc); C += oc; }
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int wm = wave / WN, wn = wave % WN;
  const int idx = blockIdx.y, q = idx & 3, j = (idx >> 2) % TN, i = (idx >> 2) / TN;
  const LongType tileLinear = (bz * tilesM + tm) * tilesN + tn;
  const LongType col = n0 + wn * WTN + j * 32 + (lane & 31);
  const LongType row0 = m0 + wm * WTM + i * 32 + 8 * q + 4 * (lane >> 5);
  if (col >= g.N || row0 >= g.M) return;
  const f32x4v* src = reinterpret_cast<const f32x4v*>(g.partial) + tileLinear * g.splits * (LongType)(Q * NT) + idx * NT + t;
  f32x4v tot = {0.f, 0.f, 0.f, 0.f};
  for (int sp0 = 0; sp0 < g.splits; sp0 += 8) {
    f32x4v v[8];
#pragma unroll
    for (int u = 0; u < 8; u++) {
      v[u] = f32x4v{0.f, 0.f, 0.f, 0.f};
      if (sp0 + u < g.splits) v[u] = src[(LongType)(sp0 + u) * (Q * NT)];
    }
#pragma unroll
    for (int u = 0; u < 8; u++) tot += v[u];
  }
#pragma unroll
  for (int e = 0; e < 4; e++) {
    if (row0 + e >= g.M) break;
    const LongType off = (row0 + e) * g.cRow + col * g.cCol;
    float v = g.alpha * tot[e];
    if (g.beta != 0.f) v += g.beta * to_float(C[off]);
    if (g.bias) v += to_float(static_cast<const T*>(g.bias)[col]);
    const T yv = Conv<T>::from(v);
    C[off] = yv;
    epilogueExtras<T>(g, row0 + e, col, yv);
  }
}

// STREAM_B: B comes through non-temporal loads (the host asks for it when the product has one row of tiles, so that every
// element of B is read exactly once, and B is large against the last-level cache)
template <typename T, int BM, int BN, int WM, int WN, bool A_KC, bool B_KC, bool STREAM_B = false>
__global__ __launch_bounds__(WM * WN * 64) void gemm_mfma16p(GemmArgs g, const T* __restrict__ A, const T* __restrict__ B, T* __restrict__ C,
                                                             unsigned tilesM, unsigned tilesN) {
  constexpr int BK = 64, NT = WM * WN * 64;
  constexpr int WTM = BM / WM, WTN = BN / WN, TM = WTM / 32, TN = WTN / 32;
  using LayA = TileLayout<BM, A_KC>;
  using LayB = TileLayout<BN, B_KC>;
  constexpr int SLOTS_A = LayA::SLOTS, SLOTS_B = LayB::SLOTS, STAGE = SLOTS_A + SLOTS_B;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  u32x4* smem = reinterpret_cast<u32x4*>(smem_raw);

  unsigned tm, tn;
  tileOf(blockIdx.x, gridDim.x, tilesM, tilesN, tm, tn);
  const LongType m0 = (LongType)tm * BM, n0 = (LongType)tn * BN;
  const LongType bz = blockIdx.z;
  { LongType oa, ob, oc; batchOffsets(g, bz, oa, ob, oc); A += oa; B += ob; C += oc; }
  const LongType lda = A_KC ? g.aRow : g.aCol, ldb = B_KC ? g.bCol : g.bRow;

  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int wm = wave / WN, wn = wave % WN;

  f32x16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int j = 0; j < TN; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

  TileLoader<BM, NT, A_KC> la;
  TileLoader<BN, NT, B_KC> lb;
  const LongType KT = (g.K + BK - 1) / BK;

  la.load(A, lda, m0, g.M, 0, g.K, t);
  lb.template load<T, STREAM_B>(B, ldb, n0, g.N, 0, g.K, t);
  la.store(smem, t);
  lb.store(smem + SLOTS_A, t);
  __syncthreads();

  for (LongType kt = 0; kt < KT; kt++) {
    const int cur = (int)(kt & 1);
    if (kt + 1 < KT) {
      la.load(A, lda, m0, g.M, (kt + 1) * BK, g.K, t);
      lb.template load<T, STREAM_B>(B, ldb, n0, g.N, (kt + 1) * BK, g.K, t);
    }
    const u32x4* sA = smem + cur * STAGE;
    const u32x4* sB = sA + SLOTS_A;
    // software pipeline over the four k-steps: fragments of step ks+1 are read while the MFMAs of step ks
    // run; the next tile's registers are written to the other LDS stage in the shadow of step 2
    u32x4 fa[2][TM], fb[2][TN];
    auto readFrag = [&](int ks, int buf) {
      const int kg = ks * 2 + (lane >> 5);
#pragma unroll
      for (int i = 0; i < TM; i++) fa[buf][i] = sA[LayA::slot(kg, wm * WTM + i * 32 + (lane & 31))];
#pragma unroll
      for (int j = 0; j < TN; j++) fb[buf][j] = sB[LayB::slot(kg, wn * WTN + j * 32 + (lane & 31))];
    };
    readFrag(0, 0);
#pragma unroll
    for (int ks = 0; ks < BK / 16; ks++) {
      if (ks + 1 < BK / 16) readFrag(ks + 1, (ks + 1) & 1);
      if (ks == 2 && kt + 1 < KT) {
        u32x4* dst = smem + (cur ^ 1) * STAGE;
        la.store(dst, t);
        lb.store(dst + SLOTS_A, t);
      }
#pragma unroll
      for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++) acc[i][j] = Mfma16<T>::mma(fa[ks & 1][i], fb[ks & 1][j], acc[i][j]);
      // interleave: one LDS read issued per pair of MFMAs
#pragma unroll
      for (int q = 0; q < (TM + TN); q++) {
        __builtin_amdgcn_sched_group_barrier(0x008, (TM * TN) / (TM + TN) > 0 ? (TM * TN) / (TM + TN) : 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
    }
    __syncthreads();
  }

  storeAccTiles<T, TM, TN, true>(g, C, acc, m0 + wm * WTM, n0 + wn * WTN, lane);
}

// The same kernel with the global loads of PD K-tiles in flight (PD register sets, the K loop unrolled PD times so that
// each set is a fixed group of registers): for launches that put one small tile on a CU, where a K-tile's MFMAs take
// 130 cycles and the loop otherwise runs at one memory latency per K-tile.  Whole tiles only, K a multiple of PD K-tiles.
template <typename T, int BM, int BN, int WM, int WN, bool A_KC, bool B_KC, int PD>
__global__ __launch_bounds__(WM * WN * 64) void gemm_mfma16q(GemmArgs g, const T* __restrict__ A, const T* __restrict__ B, T* __restrict__ C,
                                                             unsigned tilesM, unsigned tilesN) {
  constexpr int BK = 64, NT = WM * WN * 64;
  constexpr int WTM = BM / WM, WTN = BN / WN, TM = WTM / 32, TN = WTN / 32;
  using LayA = TileLayout<BM, A_KC>;
  using LayB = TileLayout<BN, B_KC>;
  constexpr int SLOTS_A = LayA::SLOTS, SLOTS_B = LayB::SLOTS, STAGE = SLOTS_A + SLOTS_B;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  u32x4* smem = reinterpret_cast<u32x4*>(smem_raw);

  unsigned tm, tn;
  tileOf(blockIdx.x, gridDim.x, tilesM, tilesN, tm, tn);
  const LongType m0 = (LongType)tm * BM, n0 = (LongType)tn * BN;
  const LongType bz = blockIdx.z;
  { LongType oa, ob, oc; batchOffsets(g, bz, oa, ob, oc); A += oa; B += ob; C += oc; }
  const LongType lda = A_KC ? g.aRow : g.aCol, ldb = B_KC ? g.bCol : g.bRow;

  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int wm = wave / WN, wn = wave % WN;

  f32x16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int j = 0; j < TN; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

  static_assert(PD % 2 == 0, "the LDS stage of a K-tile must be a compile-time constant inside the unrolled loop");
  // B with unit column stride stays in LDS as it lies in memory and is read with the transposing LDS read; transposed in
  // registers on the way in (v_perm_b32, eight 8-byte stores per thread) it cost 1.7 us of a 1024^3 launch
  using LoaderB = std::conditional_t<B_KC, TileLoader<BN, NT, true>, RowTileLoader<BN, NT>>;
  TileLoader<BM, NT, A_KC> la[PD];
  LoaderB lb[PD];
  const LongType KT = (g.K + BK - 1) / BK;

  // K is a multiple of PD K-tiles (host), and nothing below is conditional: loads past the end re-read the last K-tile and
  // the store after the last K-tile writes a stage nobody reads.  The K loop is then one basic block, which is what lets
  // the compiler wait for exactly one register set while the younger loads stay in flight.
#pragma unroll
  for (int u = 0; u < PD; u++) {
    la[u].loadFull(A, lda, m0, (LongType)u * BK, t);
    lb[u].loadFull(B, ldb, n0, (LongType)u * BK, t);
  }
  la[0].store(smem, t);
  lb[0].store(smem + SLOTS_A, t);
  __syncthreads();

  // All four k-steps' fragments of a K-tile are held in registers, and those of K-tile kt + 1 are read right after the
  // barrier that completes its stage, under the MFMAs of K-tile kt.  With one wave per SIMD and one accumulator per wave
  // there is nothing else to cover an LDS round trip: reading the fragments one k-step ahead of their MFMA (32 cycles
  // of cover for a latency several times that) made every k-step wait, 750 cycles per K-tile where the L2 stream of the
  // tile takes about 410.
  u32x4 fa[2][BK / 16][TM], fb[2][BK / 16][TN];
  int trB[TN];
#pragma unroll
  for (int j = 0; j < TN; j++) trB[j] = B_KC ? 0 : RowTileLoader<BN, NT>::fragOffset(wn * WTN + j * 32, lane);
  auto readTile = [&](int stage, int buf) {
    const u32x4* sA = smem + stage * STAGE;
    const u32x4* sB = sA + SLOTS_A;
#pragma unroll
    for (int ks = 0; ks < BK / 16; ks++) {
      const int kg = ks * 2 + (lane >> 5);
#pragma unroll
      for (int i = 0; i < TM; i++) fa[buf][ks][i] = sA[LayA::slot(kg, wm * WTM + i * 32 + (lane & 31))];
#pragma unroll
      for (int j = 0; j < TN; j++) {
        if constexpr (B_KC) fb[buf][ks][j] = sB[LayB::slot(kg, wn * WTN + j * 32 + (lane & 31))];
        else fb[buf][ks][j] = RowTileLoader<BN, NT>::readFrag(sB, trB[j], ks);
      }
    }
  };
  readTile(0, 0);

  for (LongType kt0 = 0; kt0 < KT; kt0 += PD) {
#pragma unroll
  for (int u = 0; u < PD; u++) {
    const LongType kt = kt0 + u;
    const int cur = u & 1;
    // K-tile kt + 1 leaves its registers for the other stage (whose fragments every wave read before the last barrier)
    {
      u32x4* dst = smem + (cur ^ 1) * STAGE;
      la[(u + 1) % PD].store(dst, t);
      lb[(u + 1) % PD].store(dst + SLOTS_A, t);
    }
    // K-tile kt went to LDS one round ago: its register set takes K-tile kt + PD
    {
      const LongType nx = kt + PD < KT ? kt + PD : KT - 1;
      la[u].loadFull(A, lda, m0, nx * BK, t);
      lb[u].loadFull(B, ldb, n0, nx * BK, t);
    }
    __syncthreads();
    readTile(cur ^ 1, cur ^ 1);
#pragma unroll
    for (int ks = 0; ks < BK / 16; ks++)
#pragma unroll
      for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++) acc[i][j] = Mfma16<T>::mma(fa[cur][ks][i], fb[cur][ks][j], acc[i][j]);
  }
  }

  storeAccTiles<T, TM, TN, true>(g, C, acc, m0 + wm * WTM, n0 + wn * WTN, lane);
}

// What a lane of a direct-load kernel reads for the part of an operand that lies beyond K (their KTAIL instantiations).
__device__ __attribute__((aligned(256))) unsigned char gemmZeroPage[256];

// Small tiles (64 x 64 or 128 x 128, four waves of TW x TW accumulator tiles) with the operands going from global memory
// straight into LDS (no registers, no LDS stores), NST stages in a ring: for launches that put one or two tiles on a CU
// (1024^3, 2048^3; the projections of a prefill), where the register-staged kernels spend more on parking the tiles in LDS
// than on multiplying them.  A k-contiguous, B either way; whole tiles, K a multiple of NST K-tiles.  A wave instruction moves
// a chunk of 1 KiB (64 slots of 16 bytes in lane order): 8 rows x 128 bytes of a k-contiguous operand, placed so that the
// fragment read of 32 consecutive rows is free of bank conflicts (the placement of gemm_mfma16d), or whole k-rows of
// row-major B, swizzled as RowTileLoader keeps them and read with the transposing LDS read.  Round kt: wait for tile kt + 1
// (this wave's chunks), barrier (everybody's), refill the stage tile kt - 1 left, read the fragments of tile kt + 1 while the
// MFMAs of tile kt run.
// EDGE: M and N need not be whole tiles -- rows (16-byte column groups of a row-major B) beyond the edge are read from
// clamped positions inside the operand and only reach elements of C that the bounds-checked store leaves out.
// KTAIL: K need not be a whole number of K-tiles (a multiple of 8 where an operand is k-contiguous).  Along K the products
// beyond the edge must be zero: a lane whose 16 bytes start at k >= K reads them from a page of zeros instead (same
// instruction, another address), so the loop and the LDS layouts do not change; the rounds past the last K-tile of an
// NST-round multiply zeros.
// A_KC = false: A lies [k][m] with unit m stride (a transposed A) and is handled like a row-major B: whole k-rows in LDS,
// fragments through the transposing read.
// SPLIT (with EDGE and KTAIL): blockIdx.y owns g.ktPerSplit K-tiles and parks its tile for splitk_finish; what lies beyond its
// range of K comes from the page of zeros like what lies beyond K.
template <typename T, bool B_KC, int NST, int TW, bool EDGE = false, bool KTAIL = false, bool A_KC = true, bool SPLIT = false>
__global__ __launch_bounds__(256) void gemm_mfma16s(GemmArgs g, const T* __restrict__ A, const T* __restrict__ B, T* __restrict__ C,
                                                    unsigned tilesM, unsigned tilesN) {
  constexpr int BM = 64 * TW, BN = 64 * TW, BK = 64;
  constexpr int SLOTS_A = BM * 8, STAGE = (BM + BN) * 8;   // slots of 16 bytes
  constexpr int CPW = BM / 32;                             // chunks per wave and operand
  typedef __attribute__((address_space(3))) void* lds_ptr;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  u32x4* smem = reinterpret_cast<u32x4*>(smem_raw);
  unsigned tm, tn;
  tileOf(blockIdx.x, gridDim.x, tilesM, tilesN, tm, tn);
  const LongType m0 = (LongType)tm * BM, n0 = (LongType)tn * BN;
  { LongType oa, ob, oc; batchOffsets(g, (LongType)blockIdx.z, oa, ob, oc); A += oa; B += ob; C += oc; }
  const LongType lda = A_KC ? g.aRow : g.aCol, ldb = B_KC ? g.bCol : g.bRow;
  const int t = threadIdx.x, lane = t & 63, wave = __builtin_amdgcn_readfirstlane(t >> 6), h = lane >> 5;
  const int wm = wave >> 1, wn = wave & 1;
  using RowB = RowTileLoader<BN, 256>;
  using RowA = RowTileLoader<BM, 256>;

  // ---- global side: CPW chunks of each operand per wave; a load is scalar base (the tile's first byte) + lane offset ----
  unsigned offA[CPW], offB[CPW];
  int kA[CPW], kB[CPW];   // KTAIL: the k (inside a K-tile) this lane's 16 bytes start at
#pragma unroll
  for (int c = 0; c < CPW; c++) {
    const int cw = wave * CPW + c, lj = lane >> 3, lp = lane & 7;
    const int lkg = (lp - 4 * (cw & 1) - (lj >> 1)) & 7;
    kA[c] = A_KC ? lkg * 8 : cw * (64 / RowA::SPR) + lane / RowA::SPR;
    kB[c] = B_KC ? lkg * 8 : cw * (64 / RowB::SPR) + lane / RowB::SPR;
    if (A_KC) {
      LongType ar = cw * 8 + lj;
      if (EDGE) ar = m0 + ar < g.M ? ar : g.M - 1 - m0;
      offA[c] = (unsigned)((ar * lda + lkg * 8) * 2);
    } else {
      const int k = cw * (64 / RowA::SPR) + lane / RowA::SPR, pp = lane % RowA::SPR;
      LongType ac = (pp ^ RowA::swz(k)) * 8;
      if (EDGE) ac = m0 + ac + 8 <= g.M ? ac : g.M - 8 - m0;
      offA[c] = (unsigned)(((LongType)k * lda + ac) * 2);
    }
    if (B_KC) {
      LongType br = cw * 8 + lj;
      if (EDGE) br = n0 + br < g.N ? br : g.N - 1 - n0;
      offB[c] = (unsigned)((br * ldb + lkg * 8) * 2);
    } else {
      const int k = cw * (64 / RowB::SPR) + lane / RowB::SPR, pp = lane % RowB::SPR;
      LongType bc = (pp ^ RowB::swz(k)) * 8;
      if (EDGE) bc = n0 + bc + 8 <= g.N ? bc : g.N - 8 - n0;
      offB[c] = (unsigned)(((LongType)k * ldb + bc) * 2);
    }
  }
  const char* const baseA = reinterpret_cast<const char*>(A_KC ? A + m0 * lda : A + m0);
  const char* const baseB = reinterpret_cast<const char*>(B_KC ? B + n0 * ldb : B + n0);
  const LongType stepA = (A_KC ? (LongType)BK : (LongType)BK * lda) * 2, stepB = (B_KC ? (LongType)BK : (LongType)BK * ldb) * 2;   // bytes per K-tile
  static_assert(!SPLIT || (EDGE && KTAIL && TW == 1), "the split-K instantiation handles every edge");
  const LongType ktBase = SPLIT ? (LongType)blockIdx.y * g.ktPerSplit : 0;   // first K-tile of this block
  const LongType KT = SPLIT ? g.ktPerSplit : KTAIL ? (g.K + BK - 1) / BK : g.K / BK;
  const int kEnd = SPLIT ? (int)((ktBase + g.ktPerSplit) * BK < g.K ? (ktBase + g.ktPerSplit) * BK : g.K) : (int)g.K;
  auto dma = [&](const char* base, unsigned off, const u32x4* dst) {
    const unsigned ldsAddr = (unsigned)(size_t)(lds_ptr)dst;
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(off), "s"(base), "s"(ldsAddr) : "memory");
  };
  auto dmaAt = [&](const char* src, const u32x4* dst) {   // a full address per lane
    const unsigned ldsAddr = (unsigned)(size_t)(lds_ptr)dst;
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(src), "s"(ldsAddr) : "memory");
  };
  auto issue = [&](LongType tile, int stage) {   // tiles past the end re-read the last one into a stage nobody reads
    u32x4* const st = smem + stage * STAGE;
    if constexpr (KTAIL) {
      // any tile, also past the end: zeros for everything from K on
      const char* const zero = reinterpret_cast<const char*>(gemmZeroPage);
      const LongType gt = tile + ktBase;
      const int k0 = (int)(gt * BK);
#pragma unroll
      for (int c = 0; c < CPW; c++) dmaAt(k0 + kA[c] < kEnd ? baseA + gt * stepA + offA[c] : zero, st + (wave * CPW + c) * 64);
#pragma unroll
      for (int c = 0; c < CPW; c++) dmaAt(k0 + kB[c] < kEnd ? baseB + gt * stepB + offB[c] : zero, st + SLOTS_A + (wave * CPW + c) * 64);
      return;
    }
    const LongType kt = tile < KT ? tile : KT - 1;
#pragma unroll
    for (int c = 0; c < CPW; c++) dma(baseA + kt * stepA, offA[c], st + (wave * CPW + c) * 64);
#pragma unroll
    for (int c = 0; c < CPW; c++) dma(baseB + kt * stepB, offB[c], st + SLOTS_A + (wave * CPW + c) * 64);
  };

  // ---- LDS side ----
  int fragA[TW][4], fragB[TW][4], trB[TW], trA[TW];
#pragma unroll
  for (int i = 0; i < TW; i++) {
    trA[i] = RowA::fragOffset(wm * 32 * TW + i * 32, lane);
    const int r = wm * 32 * TW + i * 32 + (lane & 31);
#pragma unroll
    for (int ks = 0; ks < 4; ks++) fragA[i][ks] = (r >> 3) * 64 + 8 * (r & 7) + ((2 * ks + h + 4 * ((r >> 3) & 1) + ((r & 7) >> 1)) & 7);
    const int rb = wn * 32 * TW + i * 32 + (lane & 31);
#pragma unroll
    for (int ks = 0; ks < 4; ks++)
      fragB[i][ks] = SLOTS_A + (rb >> 3) * 64 + 8 * (rb & 7) + ((2 * ks + h + 4 * ((rb >> 3) & 1) + ((rb & 7) >> 1)) & 7);
    trB[i] = RowB::fragOffset(wn * 32 * TW + i * 32, lane);
  }
  u32x4 fa[2][4][TW], fb[2][4][TW];
  auto readTile = [&](int stage, int buf) {
    const u32x4* st = smem + stage * STAGE;
#pragma unroll
    for (int ks = 0; ks < 4; ks++)
#pragma unroll
      for (int i = 0; i < TW; i++) {
        if (A_KC) fa[buf][ks][i] = st[fragA[i][ks]];
        else fa[buf][ks][i] = RowA::readFrag(st, trA[i], ks);
        if (B_KC) fb[buf][ks][i] = st[fragB[i][ks]];
        else fb[buf][ks][i] = RowB::readFrag(st + SLOTS_A, trB[i], ks);
      }
  };
  f32x16 acc[TW][TW];
#pragma unroll
  for (int i = 0; i < TW; i++)
#pragma unroll
    for (int j = 0; j < TW; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

  // tiles 0 .. NST - 2 on their way; tile 0 read before the loop
#pragma unroll
  for (int u = 0; u < NST - 1; u++) issue(u, u);
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"((NST - 2) * 2 * CPW) : "memory");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_sched_barrier(0);
  readTile(0, 0);
  for (LongType kt0 = 0; kt0 < KT; kt0 += NST) {
#pragma unroll
    for (int u = 0; u < NST; u++) {
      // tile kt0 + u + 1 has landed (the loads of the NST - 3 tiles after it may still be out) and is visible after the barrier
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"((NST - 3) * 2 * CPW) : "memory");
      __builtin_amdgcn_s_barrier();
      __builtin_amdgcn_sched_barrier(0);
      issue(kt0 + u + NST - 1, (u + NST - 1) % NST);   // the stage of tile kt0 + u - 1: everybody is past its fragments
      readTile((u + 1) % NST, (u + 1) & 1);
#pragma unroll
      for (int ks = 0; ks < 4; ks++)
#pragma unroll
        for (int i = 0; i < TW; i++)
#pragma unroll
          for (int j = 0; j < TW; j++) acc[i][j] = Mfma16<T>::mma(fa[u & 1][ks][i], fb[u & 1][ks][j], acc[i][j]);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the surplus loads of the last rounds
  if constexpr (SPLIT) {
    storePartialTile<TW, TW, 256>(g, acc, ((LongType)blockIdx.z * tilesM + tm) * tilesN + tn, m0 + wm * 32 * TW, n0 + wn * 32 * TW, t, lane);
    return;
  }
  if (EDGE && (m0 + BM > g.M || n0 + BN > g.N)) storeAccTiles<T, TW, TW, true>(g, C, acc, m0 + wm * 32 * TW, n0 + wn * 32 * TW, lane);
  else storeAccTiles<T, TW, TW, false>(g, C, acc, m0 + wm * 32 * TW, n0 + wn * 32 * TW, lane);
}

// Steady-state kernel for problems made of whole tiles (M % BM == 0, N % BN == 0, K % 64 == 0): no bounds handling,
// so the K loop is one basic block and the instruction order below is the order the hardware sees.  A wave issues
// in order, and an MFMA 32x32x16 keeps the matrix pipe busy for 32 cycles: every LDS / global instruction is placed
// between two MFMAs, so that its issue and its latency sit in the shadow of matrix work.
//   k-steps 0..2: fragments of the following step <- LDS                                    | 8 MFMAs each
//   k-step 3    : registers holding K-tile kt+1 -> other LDS stage                           | 4 MFMAs
//                 barrier; fragments of step 0 of tile kt+1 <- LDS; global loads of tile kt+2 | 4 MFMAs
// Global loads therefore stay in flight for a whole K-tile (about 2000 cycles) before they are needed.
template <typename T, int BM, int BN, int WM, int WN, bool A_KC, bool B_KC>
__global__ __launch_bounds__(WM * WN * 64) void gemm_mfma16f(GemmArgs g, const T* __restrict__ A, const T* __restrict__ B, T* __restrict__ C,
                                                             unsigned tilesM, unsigned tilesN) {
  constexpr int BK = 64, NT = WM * WN * 64;
  constexpr int WTM = BM / WM, WTN = BN / WN, TM = WTM / 32, TN = WTN / 32, NF = TM + TN, NM = TM * TN;
  using LayA = TileLayout<BM, A_KC>;
  using LayB = TileLayout<BN, B_KC>;
  constexpr int SLOTS_A = LayA::SLOTS, SLOTS_B = LayB::SLOTS, STAGE = SLOTS_A + SLOTS_B;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  u32x4* smem = reinterpret_cast<u32x4*>(smem_raw);

  unsigned tm, tn;
  tileOf(blockIdx.x, gridDim.x, tilesM, tilesN, tm, tn);
  const LongType m0 = (LongType)tm * BM, n0 = (LongType)tn * BN;
  const LongType bz = blockIdx.z;
  { LongType oa, ob, oc; batchOffsets(g, bz, oa, ob, oc); A += oa; B += ob; C += oc; }
  const LongType lda = A_KC ? g.aRow : g.aCol, ldb = B_KC ? g.bCol : g.bRow;
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int wm = wave / WN, wn = wave % WN;

  f32x16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int j = 0; j < TN; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

  TileLoader<BM, NT, A_KC> la;
  TileLoader<BN, NT, B_KC> lb;
  const LongType KT = g.K / BK;
  u32x4 fa[2][TM], fb[2][TN];
  // lane's fragment slots inside a stage, per k-step parity of (lane >> 5)
  int offA[TM], offB[TN];
#pragma unroll
  for (int i = 0; i < TM; i++) offA[i] = LayA::slot(lane >> 5, wm * WTM + i * 32 + (lane & 31));
#pragma unroll
  for (int j = 0; j < TN; j++) offB[j] = SLOTS_A + LayB::slot(lane >> 5, wn * WTN + j * 32 + (lane & 31));
  auto readFrag = [&](const u32x4* stage, int ks, int buf) {
#pragma unroll
    for (int i = 0; i < TM; i++) fa[buf][i] = stage[offA[i] + ks * 2 * LayA::GROUP];
#pragma unroll
    for (int j = 0; j < TN; j++) fb[buf][j] = stage[offB[j] + ks * 2 * LayB::GROUP];
  };
  auto mfmas = [&](int buf, int from, int to) {
#pragma unroll
    for (int idx = from; idx < to; idx++) {
      const int i = idx / TN, j = idx % TN;
      acc[i][j] = Mfma16<T>::mma(fa[buf][i], fb[buf][j], acc[i][j]);
    }
  };

  la.loadFull(A, lda, m0, 0, t);
  lb.loadFull(B, ldb, n0, 0, t);
  la.store(smem, t);
  lb.store(smem + SLOTS_A, t);
  la.loadFull(A, lda, m0, BK, t);        // K-tile 1 waits in registers (K >= 2 tiles)
  lb.loadFull(B, ldb, n0, BK, t);
  __syncthreads();
  readFrag(smem, 0, 0);

  for (LongType kt = 0; kt + 1 < KT; kt++) {
    const u32x4* cur = smem + (kt & 1) * STAGE;
    u32x4* nxt = smem + ((kt + 1) & 1) * STAGE;
    const LongType kAhead = (kt + 2 < KT ? kt + 2 : KT - 1) * BK;   // the last round fetches a tile nobody uses
    // k-step 0
    readFrag(cur, 1, 1);
    mfmas(0, 0, NM);
#pragma unroll
    for (int q = 0; q < NM; q++) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
    // k-step 1
    readFrag(cur, 2, 0);
    mfmas(1, 0, NM);
#pragma unroll
    for (int q = 0; q < NM; q++) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
    // k-step 2
    readFrag(cur, 3, 1);
    mfmas(0, 0, NM);
#pragma unroll
    for (int q = 0; q < NM; q++) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
    // k-step 3, first half: the registers (K-tile kt + 1, in flight for a whole tile) go to the other stage
    la.store(nxt, t);
    lb.store(nxt + SLOTS_A, t);
    mfmas(1, 0, NM / 2);
#pragma unroll
    for (int q = 0; q < NM / 2; q++) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x002, 8, 0);   // the transposing store's permutes
      __builtin_amdgcn_sched_group_barrier(0x200, 4, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();
    __builtin_amdgcn_sched_barrier(0);
    // second half: first fragments of the next tile, global loads of the tile after it
    readFrag(nxt, 0, 0);
    la.loadFull(A, lda, m0, kAhead, t);
    lb.loadFull(B, ldb, n0, kAhead, t);
    mfmas(1, NM / 2, NM);
#pragma unroll
    for (int q = 0; q < NM / 2; q++) {
      __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x020, 2, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
  }
  {
    // last K-tile: nothing left to fetch
    const u32x4* cur = smem + ((KT - 1) & 1) * STAGE;
#pragma unroll
    for (int ks = 0; ks < BK / 16; ks++) {
      if (ks + 1 < BK / 16) readFrag(cur, ks + 1, (ks + 1) & 1);
      mfmas(ks & 1, 0, NM);
#pragma unroll
      for (int q = 0; q < NM; q++) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  }

  storeAccTiles<T, TM, TN, false>(g, C, acc, m0 + wm * WTM, n0 + wn * WTN, lane);
}

// Whole-tile kernel whose global loads write LDS directly (global_load_lds_dwordx4): no staging registers, no LDS
// write instructions, and the data of K-tile kt+2 travels while tile kt is multiplied.  A wave-wide load deposits
// its 64 x 16 bytes contiguously in lane order, so the LDS layouts are chosen per lane on the global side:
//   k-contiguous operand (A, transposed B): a 1 KiB chunk holds 8 rows x 8 k-groups (8 k each), i.e. the whole
//     128-byte line of each row; slot 8j + p of chunk q holds row j, k-group (p - 4 (q%2) - j/2) % 8.  Eight
//     neighbouring lanes fetch one full line, and the 16 rows a fragment read touches per LDS pass fall into 16
//     different 16-byte bank groups.
//   row-major B ([k][n], n contiguous): a 1 KiB chunk holds two k-rows of 256 n; the 16-byte column group c of row k
//     sits at position c ^ 4 (k % 4).  Fragments come out of LDS through the transposing read ds_read_b64_tr_b16:
//     in a group of 16 lanes, lane R hands in the address of B[k0 + R/4][n0 + 4 (R%4) ..+3] and lane i receives
//     B[k0 .. k0+3][n0 + i] -- 16 columns x 4 k per read, two reads per MFMA operand.
// Two LDS stages of 64 KiB.  Per K-tile: k-steps 0..2 prefetch the next step's fragments; k-step 3 runs half of its
// MFMAs, waits for the direct loads of tile kt+1, meets the barrier, then reads the first fragments of tile kt+1 and
// issues the direct loads of tile kt+2 into the stage that was just drained.
// EDGE: M and N need not be whole tiles.  The direct loads of the last tile row / column take their rows (their 16-byte
// column groups of a row-major B) from clamped positions inside the operand -- what they bring in only ever reaches
// elements of C beyond the edge, which the bounds-checked store leaves out.
// KTAIL: K need not be a whole number of K-tiles -- lanes whose 16 bytes start at k >= K read a page of zeros (see
// gemm_mfma16s).
// A_KC = false: A lies [k][m] with unit m stride (a transposed A) and takes the row-major path of B on its side.
template <typename T, bool B_KC, bool EDGE = false, bool KTAIL = false, bool A_KC = true>
__global__ __launch_bounds__(512) void gemm_mfma16d(GemmArgs g, const T* __restrict__ A, const T* __restrict__ B, T* __restrict__ C,
                                                    unsigned tilesM, unsigned tilesN) {
  constexpr int BM = 256, BN = 256, BK = 64, WN = 4, WTM = 128, WTN = 64, TM = 4, TN = 2, NM = TM * TN;
  constexpr int SLOTS_OP = 256 * 8;              // 16-byte slots of one operand tile (32 KiB)
  constexpr int STAGE = 2 * SLOTS_OP;
  typedef __attribute__((address_space(3))) void* lds_ptr;
  typedef const __attribute__((address_space(1))) void* glb_ptr;
  typedef short s16x4 __attribute__((ext_vector_type(4)));
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  u32x4* smem = reinterpret_cast<u32x4*>(smem_raw);

  unsigned tm, tn;
  tileOf(blockIdx.x, gridDim.x, tilesM, tilesN, tm, tn);
  const LongType m0 = (LongType)tm * BM, n0 = (LongType)tn * BN;
  const LongType bz = blockIdx.z;
  { LongType oa, ob, oc; batchOffsets(g, bz, oa, ob, oc); A += oa; B += ob; C += oc; }
  const LongType lda = A_KC ? g.aRow : g.aCol, ldb = B_KC ? g.bCol : g.bRow;
  const int t = threadIdx.x, lane = t & 63, wave = __builtin_amdgcn_readfirstlane(t >> 6), h = lane >> 5;
  const int wm = wave / WN, wn = wave % WN;

  // ---- global side: this wave's four chunks of each operand ------------------------------------------------------
  // k-contiguous operand, chunk id cw = wave * 4 + i: rows cw * 8 .. +7, all 8 k-groups (a whole 128-byte line per row)
  const int lj = lane >> 3, lp = lane & 7;
  const T* aSrc[4];
  const T* bSrc[4];
  int akg[4], bkg[4];   // KTAIL: the k (inside a K-tile) this lane's 16 bytes start at
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const int cw = wave * 4 + i;
    const int lkg = (lp - 4 * (cw & 1) - (lj >> 1)) & 7;
    akg[i] = A_KC ? lkg * 8 : 2 * cw + (lane >> 5);
    bkg[i] = B_KC ? lkg * 8 : 2 * cw + (lane >> 5);
    if (A_KC) {
      LongType ar = m0 + cw * 8 + lj;
      if (EDGE) ar = ar < g.M ? ar : g.M - 1;
      aSrc[i] = A + ar * lda + lkg * 8;
    } else {
      const int kr = 2 * cw + (lane >> 5), q = lane & 31, c = q ^ (4 * (kr & 3));
      LongType ac = m0 + 8 * c;
      if (EDGE) ac = ac + 8 <= g.M ? ac : g.M - 8;
      aSrc[i] = A + (LongType)kr * lda + ac;
    }
    if (B_KC) {
      LongType br = n0 + cw * 8 + lj;
      if (EDGE) br = br < g.N ? br : g.N - 1;
      bSrc[i] = B + br * ldb + lkg * 8;
    } else {
      const int kr = 2 * cw + (lane >> 5), q = lane & 31, c = q ^ (4 * (kr & 3));
      LongType bc = n0 + 8 * c;
      if (EDGE) bc = bc + 8 <= g.N ? bc : g.N - 8;
      bSrc[i] = B + (LongType)kr * ldb + bc;
    }
  }
  const LongType aStep = A_KC ? (LongType)BK : (LongType)BK * lda, bStep = B_KC ? (LongType)BK : (LongType)BK * ldb;
  // The loads are written as assembly on purpose.  Issued through the builtin, the compiler's wait-count pass knows of
  // an outstanding write into LDS and, having no alias information for the transposing read, puts s_waitcnt vmcnt(0)
  // in front of every ds_read_b64_tr_b16 that follows -- twice per K-tile the wave then sits out the whole latency of
  // loads it has only just issued.  All waiting on these loads is explicit in this kernel (s_waitcnt vmcnt before the
  // barrier), so the compiler need not know of them.  M0 carries the LDS address of the wave's chunk; nothing else in
  // this kernel uses M0 (it is a reserved register and cannot be named as a clobber).
  auto loadToLds = [&](const T* src, u32x4* dst) {
    const unsigned ldsAddr = (unsigned)(size_t)(lds_ptr)dst;
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(src), "s"(ldsAddr) : "memory");
  };
  int ldA = 0, ldB = 0;   // KTAIL: first k of the K-tile the next A / B loads belong to
  const T* const zero = reinterpret_cast<const T*>(gemmZeroPage);
  auto issueLoads = [&](u32x4* stage, int from, int to) {
#pragma unroll
    for (int i = from; i < to; i++) {
      if (i < 4) {
        loadToLds(!KTAIL || ldA + akg[i] < (int)g.K ? aSrc[i] : zero, stage + (wave * 4 + i) * 64);
        aSrc[i] += aStep;
        if (KTAIL && i == 3) ldA += BK;
      } else {
        loadToLds(!KTAIL || ldB + bkg[i - 4] < (int)g.K ? bSrc[i - 4] : zero, stage + SLOTS_OP + (wave * 4 + i - 4) * 64);
        bSrc[i - 4] += bStep;
        if (KTAIL && i == 7) ldB += BK;
      }
    }
  };

  // ---- LDS side: fragment addresses ---------------------------------------------------------------------------------
  // k-contiguous layout: row r, k-group kg = 2 ks + h -> chunk r / 8, slot 8 (r % 8) + ((kg + 4 (r / 8 % 2) + r % 8 / 2) & 7)
  int offA[TM][4], offB[TN][4];
#pragma unroll
  for (int i = 0; i < TM; i++) {
    const int r = wm * WTM + i * 32 + (lane & 31);
#pragma unroll
    for (int ks = 0; ks < 4; ks++) offA[i][ks] = (r >> 3) * 64 + 8 * (r & 7) + ((2 * ks + h + 4 * ((r >> 3) & 1) + ((r & 7) >> 1)) & 7);
  }
  int trA[TM];   // byte offsets of the transposing reads (row-major A)
#pragma unroll
  for (int i = 0; i < TM; i++) {
    const int grp = lane >> 4, i16 = lane & 15;
    const int n4 = wm * WTM + i * 32 + 16 * (grp & 1) + 4 * (i16 & 3);
    const int k = 8 * (grp >> 1) + (i16 >> 2);
    const int phys = (n4 >> 3) ^ (4 * ((i16 >> 2) & 3));
    trA[i] = k * 512 + phys * 16 + ((n4 >> 2) & 1) * 8;
  }
  int trB[TN];   // byte offsets of the transposing reads (row-major B)
#pragma unroll
  for (int jt = 0; jt < TN; jt++) {
    if (B_KC) {
      const int r = wn * WTN + jt * 32 + (lane & 31);
#pragma unroll
      for (int ks = 0; ks < 4; ks++)
        offB[jt][ks] = SLOTS_OP + (r >> 3) * 64 + 8 * (r & 7) + ((2 * ks + h + 4 * ((r >> 3) & 1) + ((r & 7) >> 1)) & 7);
      trB[jt] = 0;
    } else {
      const int grp = lane >> 4, i16 = lane & 15;
      const int n4 = wn * WTN + jt * 32 + 16 * (grp & 1) + 4 * (i16 & 3);
      const int k = 8 * (grp >> 1) + (i16 >> 2);                       // + 16 ks + 4 rd
      const int phys = (n4 >> 3) ^ (4 * ((i16 >> 2) & 3));
      trB[jt] = SLOTS_OP * 16 + k * 512 + phys * 16 + ((n4 >> 2) & 1) * 8;
      offB[jt][0] = offB[jt][1] = offB[jt][2] = offB[jt][3] = 0;
    }
  }
  u32x4 fa[2][TM], fb[2][TN];
  auto readFrag = [&](const u32x4* stage, int ks, int buf) {
#pragma unroll
    for (int i = 0; i < TM; i++) {
      if (A_KC) {
        fa[buf][i] = stage[offA[i][ks]];
      } else {
        const __attribute__((address_space(3))) unsigned char* base =
            (const __attribute__((address_space(3))) unsigned char*)(lds_ptr)stage + trA[i] + ks * 8192;
        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)base);
        const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(base + 2048));
        const u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
        fa[buf][i] = u32x4{l2[0], l2[1], h2[0], h2[1]};
      }
    }
#pragma unroll
    for (int jt = 0; jt < TN; jt++) {
      if (B_KC) {
        fb[buf][jt] = stage[offB[jt][ks]];
      } else {
        const __attribute__((address_space(3))) unsigned char* base =
            (const __attribute__((address_space(3))) unsigned char*)(lds_ptr)stage + trB[jt] + ks * 8192;
        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)base);
        const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(base + 2048));
        const u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
        fb[buf][jt] = u32x4{l2[0], l2[1], h2[0], h2[1]};
      }
    }
  };

  f32x16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int j = 0; j < TN; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;
  auto mfmas = [&](int buf, int from, int to) {
#pragma unroll
    for (int idx = from; idx < to; idx++) {
      const int i = idx / TN, j = idx % TN;
      acc[i][j] = Mfma16<T>::mma(fa[buf][i], fb[buf][j], acc[i][j]);
    }
  };

  const LongType KT = KTAIL ? (g.K + BK - 1) / BK : g.K / BK;
  issueLoads(smem, 0, 8);            // tile 0 -> stage 0
  issueLoads(smem + STAGE, 0, 8);    // tile 1 -> stage 1 (K >= 2 tiles)
  asm volatile("s_waitcnt vmcnt(8)" ::: "memory");   // tile 0 has landed (loads complete in order)
  __syncthreads();
  readFrag(smem, 0, 0);

  // one K-tile round; LOADS: the direct loads of tile kt + 2 are issued here (second half of k-step 3) and
  // the first half of them in the NEXT round's k-step 0 -- spread out, each between two MFMAs
  auto round = [&](LongType kt, auto loadsNow, auto loadsLate) {
    u32x4* cur = smem + (kt & 1) * STAGE;
    u32x4* nxt = smem + ((kt + 1) & 1) * STAGE;
#pragma unroll
    for (int ks = 0; ks < 3; ks++) {
      readFrag(cur, ks + 1, (ks + 1) & 1);
      if (ks == 0 && decltype(loadsLate)::value) issueLoads(nxt, 4, 8);   // second half of tile kt + 1 (B operand)
      mfmas(ks & 1, 0, NM);
#pragma unroll
      for (int q = 0; q < NM; q++) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, B_KC ? 1 : 2, 0);
        if (ks == 0 && decltype(loadsLate)::value && (q & 1)) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    // k-step 3: half of the MFMAs, then tile kt + 1 must be in LDS for everybody
    mfmas(1, 0, NM / 2);
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    __builtin_amdgcn_sched_barrier(0);
    readFrag(nxt, 0, 0);
    if (decltype(loadsNow)::value) issueLoads(cur, 0, 4);   // first half of tile kt + 2 (A operand) into the drained stage
    mfmas(1, NM / 2, NM);
#pragma unroll
    for (int q = 0; q < NM / 2; q++) {
      __builtin_amdgcn_sched_group_barrier(0x100, B_KC ? 2 : 3, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      if (decltype(loadsNow)::value) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  using Yes = std::true_type;
  using No = std::false_type;
  // round kt consumes tile kt; tile kt + 1 is complete in LDS by its barrier.  Tile 1 was issued whole in the prologue.
  if (KT >= 3) {
    round(0, Yes{}, No{});
    for (LongType kt = 1; kt + 2 < KT; kt++) round(kt, Yes{}, Yes{});
    round(KT - 2, No{}, Yes{});
  } else {
    round(0, No{}, No{});
  }
  {
    const u32x4* cur = smem + ((KT - 1) & 1) * STAGE;
#pragma unroll
    for (int ks = 0; ks < BK / 16; ks++) {
      if (ks + 1 < BK / 16) readFrag(cur, ks + 1, (ks + 1) & 1);
      mfmas(ks & 1, 0, NM);
      __builtin_amdgcn_sched_barrier(0);
    }
  }

  if (EDGE && (m0 + BM > g.M || n0 + BN > g.N)) storeAccTiles<T, TM, TN, true>(g, C, acc, m0 + wm * WTM, n0 + wn * WTN, lane);
  else storeAccTiles<T, TM, TN, false>(g, C, acc, m0 + wm * WTM, n0 + wn * WTN, lane);   // a whole tile, also of a ragged product
}

// The same 256 x 256 tile for A k-contiguous and B row-major with the operands in two RINGS of LDS units instead of two
// whole stages, so that a slot is refilled as soon as it is drained and the direct loads are issued at an even rate --
// one A and one B load per wave and eight MFMAs -- with at least one step (sixteen MFMAs per wave) between a load's
// issue and the barrier that hands its data to the readers.
//   step = 32 k = two k-steps of eight MFMAs (phase 0, phase 1), one barrier per step, between the phases.
//   A ring: 3 units of 256 rows x 64 k (whole 128-byte lines of every row, chunk layout of gemm_mfma16d), 32 KiB each;
//           unit j serves steps 2j and 2j + 1.
//   B ring: 4 units of 32 k-rows x 256 n, 16 KiB each; unit s serves step s.            3 * 32 + 4 * 16 = 160 KiB.
// Phase 0 of step s reads the fragments of phase 1; phase 1 reads those of step s + 1, phase 0.  The barrier of step s
// therefore certifies (a) that the units step s + 1 reads have landed and (b) that every wave is through with the units
// of step s - 1.  What is issued when (j = s / 2; a wave owns chunks 0..3 of every A unit and chunks 0..1 of every B unit):
//   even s: phase 0: A chunk 3 of unit j + 1, B chunk 1 of unit s + 2;   phase 1: A chunk 0 of unit j + 2, B chunk 0 of unit s + 3
//   odd s:  phase 0: A chunk 1 of unit j + 2, B chunk 1 of unit s + 2;   phase 1: A chunk 2 of unit j + 2, B chunk 0 of unit s + 3
// Every load goes into a slot whose unit was last read two barriers ago, and is at least four loads old (two phases)
// when the barrier that certifies it is reached: s_waitcnt vmcnt(4) in front of every barrier (loads complete in
// order).  The loop is branch-free: past the end of K the pointers stop advancing, so the surplus loads re-read the
// last unit into slots nobody reads any more.  K must be a multiple of 128 (four steps per loop iteration).
// EDGE as in gemm_mfma16d: clamped loads and a bounds-checked store for an M or N that is not a whole number of tiles.
// KTAIL: K need not be a multiple of 128 -- the loop runs over K rounded up, and lanes whose 16 bytes start at k >= K read a
// page of zeros (see gemm_mfma16s).
template <typename T, bool EDGE = false, bool KTAIL = false>
__global__ __launch_bounds__(512) void gemm_mfma16r(GemmArgs g, const T* __restrict__ A, const T* __restrict__ B, T* __restrict__ C,
                                                    unsigned tilesM, unsigned tilesN) {
  constexpr int BM = 256, BN = 256, WN = 4, WTM = 128, WTN = 64, TM = 4, TN = 2, NM = TM * TN;
  constexpr int A_UNIT = 256 * 8;     // 16-byte slots of one A unit
  constexpr int B_UNIT = 32 * 32;     // 16-byte slots of one B unit
  constexpr int B_BASE = 3 * A_UNIT;  // the B ring sits behind the A ring
  typedef __attribute__((address_space(3))) void* lds_ptr;
  typedef short s16x4 __attribute__((ext_vector_type(4)));
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  u32x4* smem = reinterpret_cast<u32x4*>(smem_raw);

  unsigned tm, tn;
  tileOf(blockIdx.x, gridDim.x, tilesM, tilesN, tm, tn);
  const LongType m0 = (LongType)tm * BM, n0 = (LongType)tn * BN;
  { LongType oa, ob, oc; batchOffsets(g, blockIdx.z, oa, ob, oc); A += oa; B += ob; C += oc; }
  const LongType lda = g.aRow, ldb = g.bRow;
  const int t = threadIdx.x, lane = t & 63, wave = __builtin_amdgcn_readfirstlane(t >> 6), h = lane >> 5;
  const int wm = wave / WN, wn = wave % WN;

  // ---- global side ---------------------------------------------------------------------------------------------------
  const int lj = lane >> 3, lp = lane & 7;
  const T* aSrc[4];
  const T* bSrc[2];
  int aK[4], bK[2];   // KTAIL: the k this lane's next 16 bytes of the chunk start at
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const int cw = wave * 4 + i;                          // 8 rows, all 8 k-groups of the unit
    const int lkg = (lp - 4 * (cw & 1) - (lj >> 1)) & 7;
    aK[i] = lkg * 8;
    LongType ar = m0 + cw * 8 + lj;
    if (EDGE) ar = ar < g.M ? ar : g.M - 1;
    aSrc[i] = A + ar * lda + lkg * 8;
  }
#pragma unroll
  for (int c = 0; c < 2; c++) {
    const int kr = 2 * (wave * 2 + c) + (lane >> 5), q = lane & 31;   // two k-rows of 256 n per chunk
    bK[c] = kr;
    LongType bc = n0 + 8 * (q ^ (4 * (kr & 3)));
    if (EDGE) bc = bc + 8 <= g.N ? bc : g.N - 8;
    bSrc[c] = B + (LongType)kr * ldb + bc;
  }
  const int Kr = KTAIL ? (int)((g.K + 127) / 128 * 128) : (int)g.K;
  const int S = Kr / 32, nA = Kr / 64;   // steps, A units
  const LongType aStep = 64, bStep = 32 * ldb;
  const T* const zero = reinterpret_cast<const T*>(gemmZeroPage);
  auto loadToLds = [&](const T* src, u32x4* dst) {
    const unsigned ldsAddr = (unsigned)(size_t)(lds_ptr)dst;
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(src), "s"(ldsAddr) : "memory");
  };
  // chunk i of A unit `unit` into ring slot `slot`; the pointer moves on only while there is a next unit
  auto issueA = [&](int i, int slot, int unit) {
    loadToLds(!KTAIL || aK[i] < (int)g.K ? aSrc[i] : zero, smem + slot * A_UNIT + (wave * 4 + i) * 64);
    aSrc[i] += unit + 1 < nA ? aStep : 0;
    if (KTAIL) aK[i] += unit + 1 < nA ? 64 : 0;
  };
  auto issueB = [&](int c, int slot, int unit) {
    loadToLds(!KTAIL || bK[c] < (int)g.K ? bSrc[c] : zero, smem + B_BASE + slot * B_UNIT + (wave * 2 + c) * 64);
    bSrc[c] += unit + 1 < S ? bStep : 0;
    if (KTAIL) bK[c] += unit + 1 < S ? 32 : 0;
  };

  // ---- LDS side --------------------------------------------------------------------------------------------------------
  int offA[TM][4];   // slot of (row, k-step ks of the unit) inside an A unit, as in gemm_mfma16d
#pragma unroll
  for (int i = 0; i < TM; i++) {
    const int r = wm * WTM + i * 32 + (lane & 31);
#pragma unroll
    for (int ks = 0; ks < 4; ks++) offA[i][ks] = (r >> 3) * 64 + 8 * (r & 7) + ((2 * ks + h + 4 * ((r >> 3) & 1) + ((r & 7) >> 1)) & 7);
  }
  int trB[TN];       // byte offset of the transposing read inside a B unit (k-step 0, first half)
#pragma unroll
  for (int jt = 0; jt < TN; jt++) {
    const int grp = lane >> 4, i16 = lane & 15;
    const int n4 = wn * WTN + jt * 32 + 16 * (grp & 1) + 4 * (i16 & 3);
    const int k = 8 * (grp >> 1) + (i16 >> 2);
    const int phys = (n4 >> 3) ^ (4 * ((i16 >> 2) & 3));
    trB[jt] = k * 512 + phys * 16 + ((n4 >> 2) & 1) * 8;
  }
  u32x4 fa[2][TM], fb[2][TN];
  // fragments of k-step ksA (0..3) of the A unit in ring slot aSlot and k-step ksB (0..1) of the B unit in slot bSlot
  auto readFragA = [&](int aSlot, int ksA, int buf) {
    const u32x4* ua = smem + aSlot * A_UNIT;
#pragma unroll
    for (int i = 0; i < TM; i++) fa[buf][i] = ua[offA[i][ksA]];
  };
  auto readFragB = [&](int bSlot, int ksB, int buf) {
    const __attribute__((address_space(3))) unsigned char* ub =
        (const __attribute__((address_space(3))) unsigned char*)(lds_ptr)(smem + B_BASE + bSlot * B_UNIT) + ksB * 8192;
#pragma unroll
    for (int jt = 0; jt < TN; jt++) {
      const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(ub + trB[jt]));
      const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(ub + trB[jt] + 2048));
      const u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
      fb[buf][jt] = u32x4{l2[0], l2[1], h2[0], h2[1]};
    }
  };

  f32x16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int j = 0; j < TN; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;
  auto mfmas = [&](int buf, int from, int to) {
#pragma unroll
    for (int idx = from; idx < to; idx++) {
      const int i = idx / TN, j = idx % TN;
      acc[i][j] = Mfma16<T>::mma(fa[buf][i], fb[buf][j], acc[i][j]);
    }
  };

  // ---- prologue: A unit 0, B units 0 and 1, A unit 1 chunks 0..2, B unit 2 chunk 0 -----------------------------------------
#pragma unroll
  for (int i = 0; i < 4; i++) issueA(i, 0, 0);
  issueB(0, 0, 0); issueB(1, 0, 0);
  issueB(0, 1, 1); issueB(1, 1, 1);
  issueA(0, 1, 1); issueA(1, 1, 1); issueA(2, 1, 1);
  issueB(0, 2, 2);
  asm volatile("s_waitcnt vmcnt(6)" ::: "memory");   // A unit 0 and B unit 0 (the first six loads) have landed
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_sched_barrier(0);
  readFragA(0, 0, 0);
  readFragB(0, 0, 0);

  int a0 = 0, a1 = 1, a2 = 2;   // ring slots of A units j, j + 1, j + 2
  // one phase = four pairs of MFMAs; the four A reads go out with the first pair, the four B reads with the second; the
  // A load is issued in front of pair PA, the B load in front of pair PB
  auto phase = [&](auto pa, auto pb, int buf, int aSlot, int ksA, int bSlot, int ksB, int nbuf, auto&& loadA, auto&& loadB) {
    constexpr int PA = decltype(pa)::value, PB = decltype(pb)::value;
#pragma unroll
    for (int pr = 0; pr < 4; pr++) {
      if (pr == PA) loadA();
      if (pr == PB) loadB();
      if (pr == 0) readFragA(aSlot, ksA, nbuf);
      if (pr == 1) readFragB(bSlot, ksB, nbuf);
      mfmas(buf, 2 * pr, 2 * pr + 2);
      if (pr < 2) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  auto sync = [&]() {
    asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
  };
  auto mainLoop = [&](auto pa, auto pb) {
    for (int s = 0; s < S; s += 4) {
      const int j = s >> 1;
      // step s (even), B slot 0
      phase(pa, pb, 0, a0, 1, 0, 1, 1, [&] { issueA(3, a1, j + 1); }, [&] { issueB(1, 2, s + 2); });
      sync();
      phase(pa, pb, 1, a0, 2, 1, 0, 0, [&] { issueA(0, a2, j + 2); }, [&] { issueB(0, 3, s + 3); });
      // step s + 1 (odd), B slot 1
      phase(pa, pb, 0, a0, 3, 1, 1, 1, [&] { issueA(1, a2, j + 2); }, [&] { issueB(1, 3, s + 3); });
      sync();
      phase(pa, pb, 1, a1, 0, 2, 0, 0, [&] { issueA(2, a2, j + 2); }, [&] { issueB(0, 0, s + 4); });
      // step s + 2 (even), B slot 2; the A units have moved on by one: (a0, a1, a2) -> (a1, a2, a0)
      phase(pa, pb, 0, a1, 1, 2, 1, 1, [&] { issueA(3, a2, j + 2); }, [&] { issueB(1, 0, s + 4); });
      sync();
      phase(pa, pb, 1, a1, 2, 3, 0, 0, [&] { issueA(0, a0, j + 3); }, [&] { issueB(0, 1, s + 5); });
      // step s + 3 (odd), B slot 3
      phase(pa, pb, 0, a1, 3, 3, 1, 1, [&] { issueA(1, a0, j + 3); }, [&] { issueB(1, 1, s + 5); });
      sync();
      phase(pa, pb, 1, a2, 0, 0, 0, 0, [&] { issueA(2, a0, j + 3); }, [&] { issueB(0, 2, s + 6); });
      const int o0 = a0, o1 = a1;
      a0 = a2; a1 = o0; a2 = o1;   // two units on: (a0, a1, a2) -> (a2, a0, a1)
    }
  };
  // the A load goes out in front of the first pair of MFMAs of a phase, the B load in front of the third (measured: 1163
  // cycles per step against 1190 with both loads in the second half of the phase; 1024 are the MFMAs alone)
  mainLoop(std::integral_constant<int, 0>{}, std::integral_constant<int, 2>{});
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the surplus loads of the last steps

  if (EDGE && (m0 + BM > g.M || n0 + BN > g.N)) storeAccTiles<T, TM, TN, true>(g, C, acc, m0 + wm * WTM, n0 + wn * WTN, lane);
  else storeAccTiles<T, TM, TN, false>(g, C, acc, m0 + wm * WTM, n0 + wn * WTN, lane);   // a whole tile, also of a ragged product
}

// ---- 16-bit MFMA kernel for operands the vector loaders cannot take ---------------------------------------------------------
// Rows that do not start on 16-byte boundaries (a row-major [K, 50257] matrix), a contiguous extent that is not a multiple
// of 8, two non-unit strides, negative strides: the tiles are gathered element by element (2-byte loads, zero beyond the
// edges) into the k-contiguous LDS layout, and from there on it is the two-stage tile kernel.  RF ("row fast"): neighbouring
// lanes take neighbouring rows of one k -- for an operand whose unit (or smaller) stride runs along its rows; otherwise
// neighbouring lanes take neighbouring k-groups of one row.
template <int ROWS, int NT, bool RF>
struct ElementTileLoader {
  using Layout = TileLayout<ROWS, true>;
  static constexpr int UNITS = ROWS * 8, PER = UNITS / NT;
  static_assert(UNITS % NT == 0, "every thread gathers the same number of k-groups");
  u32x4 reg[PER];
  static __device__ __forceinline__ void unitOf(int u, int& kg, int& row) {
    if (RF) { row = u % ROWS; kg = u / ROWS; } else { kg = u & 7; row = u >> 3; }
  }
  template <typename T>
  __device__ __forceinline__ void load(const T* __restrict__ base, LongType rs, LongType ks, LongType row0, LongType rowLimit, LongType k0, LongType K, int t) {
#pragma unroll
    for (int i = 0; i < PER; i++) {
      int kg, row;
      unitOf(t + i * NT, kg, row);
      // every load is unconditional (positions past an edge re-read the last valid one and are zeroed afterwards): a
      // predicated load would put a wait at every join, one memory latency per element
      const LongType r = row0 + row, kb = k0 + kg * 8;
      const T* p = base + (r < rowLimit ? r : rowLimit - 1) * rs;
      unsigned e[8];
#pragma unroll
      for (int j = 0; j < 8; j++) e[j] = (unsigned)p[(kb + j < K ? kb + j : K - 1) * ks].bits;
#pragma unroll
      for (int j = 0; j < 8; j++) e[j] = (r < rowLimit && kb + j < K) ? e[j] : 0u;
      reg[i] = u32x4{e[0] | (e[1] << 16), e[2] | (e[3] << 16), e[4] | (e[5] << 16), e[6] | (e[7] << 16)};
    }
  }
  __device__ __forceinline__ void store(u32x4* __restrict__ lds, int t) {
#pragma unroll
    for (int i = 0; i < PER; i++) {
      int kg, row;
      unitOf(t + i * NT, kg, row);
      lds[Layout::slot(kg, row)] = reg[i];
    }
  }
};
template <typename T, int BM, int BN, int WM, int WN, bool A_RF, bool B_RF>
__global__ __launch_bounds__(WM * WN * 64) void gemm_mfma16u(GemmArgs g, const T* __restrict__ A, const T* __restrict__ B, T* __restrict__ C,
                                                              unsigned tilesM, unsigned tilesN) {
  constexpr int BK = 64, NT = WM * WN * 64;
  constexpr int WTM = BM / WM, WTN = BN / WN, TM = WTM / 32, TN = WTN / 32;
  using LayA = TileLayout<BM, true>;
  using LayB = TileLayout<BN, true>;
  constexpr int SLOTS_A = LayA::SLOTS, SLOTS_B = LayB::SLOTS, STAGE = SLOTS_A + SLOTS_B;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  u32x4* smem = reinterpret_cast<u32x4*>(smem_raw);
  unsigned tm, tn;
  tileOf(blockIdx.x, gridDim.x, tilesM, tilesN, tm, tn);
  const LongType m0 = (LongType)tm * BM, n0 = (LongType)tn * BN;
  { LongType oa, ob, oc; batchOffsets(g, blockIdx.z, oa, ob, oc); A += oa; B += ob; C += oc; }
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int wm = wave / WN, wn = wave % WN;
  f32x16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int j = 0; j < TN; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;
  ElementTileLoader<BM, NT, A_RF> la;
  ElementTileLoader<BN, NT, B_RF> lb;
  const LongType KT = (g.K + BK - 1) / BK;
  la.load(A, g.aRow, g.aCol, m0, g.M, 0, g.K, t);
  lb.load(B, g.bCol, g.bRow, n0, g.N, 0, g.K, t);
  la.store(smem, t);
  lb.store(smem + SLOTS_A, t);
  __syncthreads();
  for (LongType kt = 0; kt < KT; kt++) {
    const int cur = (int)(kt & 1);
    if (kt + 1 < KT) {
      la.load(A, g.aRow, g.aCol, m0, g.M, (kt + 1) * BK, g.K, t);
      lb.load(B, g.bCol, g.bRow, n0, g.N, (kt + 1) * BK, g.K, t);
    }
    const u32x4* sA = smem + cur * STAGE;
    const u32x4* sB = sA + SLOTS_A;
#pragma unroll
    for (int ks = 0; ks < BK / 16; ks++) {
      const int kg = ks * 2 + (lane >> 5);
      u32x4 fa[TM], fb[TN];
#pragma unroll
      for (int i = 0; i < TM; i++) fa[i] = sA[LayA::slot(kg, wm * WTM + i * 32 + (lane & 31))];
#pragma unroll
      for (int j = 0; j < TN; j++) fb[j] = sB[LayB::slot(kg, wn * WTN + j * 32 + (lane & 31))];
#pragma unroll
      for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++) acc[i][j] = Mfma16<T>::mma(fa[i], fb[j], acc[i][j]);
    }
    if (kt + 1 < KT) {
      u32x4* dst = smem + (cur ^ 1) * STAGE;
      la.store(dst, t);
      lb.store(dst + SLOTS_A, t);
    }
    __syncthreads();
  }
  storeAccTiles<T, TM, TN, true>(g, C, acc, m0 + wm * WTM, n0 + wn * WTN, lane);
}

// How many K-splits a launch of BM x BN tiles gets: enough to put about two blocks on every CU when the tiles alone
// cannot, bounded by the K-tiles there are and the partial-tile scratch.
template <int BM, int BN>
static int chooseSplits(const GemmArgs& g, LongType batch, LongType& ktPerSplit) {
  const LongType tiles = ((g.M + BM - 1) / BM) * ((g.N + BN - 1) / BN) * batch, KT = (g.K + 63) / 64;
  ktPerSplit = KT;
  if (tiles >= 192 || KT < 2) return 1;
  LongType want = (512 + tiles - 1) / tiles;
  want = want < KT ? want : KT;
  want = want < 16 ? want : 16;          // one finishing block reads every partial of its tile
  const LongType cap = (LongType)(LaunchContext::ALLOCATION_BYTES / sizeof(float)) / (tiles * BM * BN);
  want = want < cap ? want : cap;
  if (want < 2) return 1;
  ktPerSplit = (KT + want - 1) / want;
  return (int)((KT + ktPerSplit - 1) / ktPerSplit);
}

template <typename T, int BM, int BN, int WM, int WN, bool A_KC, bool B_KC>
static bool launchMfma16Cfg(hipStream_t s, GemmArgs g, const void* A, const void* B, void* C, LongType batch, bool allowSplit, bool aligned) {
  constexpr int NT = WM * WN * 64;
  constexpr size_t LDS = (size_t)2 * (TileLayout<BM, A_KC>::SLOTS + TileLayout<BN, B_KC>::SLOTS) * 16;
  int splits = 1;
  // 64 x 64 tiles that the direct-load ring kernel below can take, K up to 2048: one block per tile and no split beats
  // split-K plus its finishing launch even with a quarter of the CUs busy (bf16 512^3 4.5 against 11.2 us, 768^3 4.7 against
  // 12.0, 512 x 512 x 2048 7.7 against 13.0; from K = 4096 on the split wins: 256 x 256 x 4096 10.4 against 11.9)
  bool ringInstead = false;
  // the ring kernel's edge instantiation takes an M or N that is not a whole number of tiles (a row-major B in whole
  // 16-byte column groups)
  static const bool edge = getenv("ND4JHIP_GEMM_EDGE") ? atoi(getenv("ND4JHIP_GEMM_EDGE")) != 0 : true;
  const bool whole = g.M % BM == 0 && g.N % BN == 0;
  const bool edgeOk = whole || (edge && (B_KC || g.N % 8 == 0) && (A_KC || g.M % 8 == 0));
  if constexpr (BM == 64 && BN == 64 && WM == 2 && WN == 2) {
    static const bool small = getenv("ND4JHIP_GEMM_SMALL_RING") ? atoi(getenv("ND4JHIP_GEMM_SMALL_RING")) != 0 : true;
    const LongType ldaS = A_KC ? g.aRow : g.aCol, ldbS = B_KC ? g.bCol : g.bRow;
    const bool edgeRoute = edge && aligned && (!whole || g.K % 64 != 0);   // what the edge instantiation takes from K = 128 on
    ringInstead = small && (g.K >= 512 || (edgeRoute && g.K >= 128)) && g.K <= 2048 && (g.K % 256 == 0 || edgeRoute) && edgeOk && (whole || aligned) &&
                  ((g.M + BM - 1) / BM) * ((g.N + BN - 1) / BN) * batch <= 1024 &&
                  ldaS % 8 == 0 && ldbS % 8 == 0 && ldaS < (1 << 23) && ldbS < (1 << 23) &&
                  ((reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(B)) & 15) == 0 && g.aBatch % 8 == 0 && g.bBatch % 8 == 0 &&
                  g.aBatch2 % 8 == 0 && g.bBatch2 % 8 == 0 && !g.hasEpi;
  }
  if (allowSplit && !ringInstead) {
    LongType per = 0;
    splits = chooseSplits<BM, BN>(g, batch, per);
    if (splits > 1) {
      LaunchContext* lc = LaunchContext::defaultContext();
      g.splits = splits; g.ktPerSplit = per;
      g.partial = static_cast<float*>(lc->allocationBuffer);
    }
  }
  // an epilogue request is served by splitk_finish only (one batch entry, unit column stride of C)
  if (g.hasEpi && (splits == 1 || batch != 1 || g.cCol != 1)) return false;
  // split-K on the direct-load ring: few 64 x 64 tiles and a long K.  Every block keeps a whole round of K-tiles in flight,
  // where the register-staged split kernel pays one memory latency per K-tile; fewer, deeper splits (about one block per
  // CU, four K-tiles at least) leave less for the finishing launch to add up.
  if constexpr (BM == 64 && BN == 64 && WM == 2 && WN == 2) {
    static const bool small = getenv("ND4JHIP_GEMM_SMALL_RING") ? atoi(getenv("ND4JHIP_GEMM_SMALL_RING")) != 0 : true;
    static const bool splitRing = getenv("ND4JHIP_GEMM_SPLIT_RING") ? atoi(getenv("ND4JHIP_GEMM_SPLIT_RING")) != 0 : true;
    const LongType ldaS = A_KC ? g.aRow : g.aCol, ldbS = B_KC ? g.bCol : g.bRow;
    if (splits > 1 && small && splitRing && edge && aligned && (B_KC || g.N % 8 == 0) && (A_KC || g.M % 8 == 0) && ldaS % 8 == 0 && ldbS % 8 == 0 &&
        ldaS < (1 << 23) && ldbS < (1 << 23) && ((reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(B)) & 15) == 0 && g.aBatch % 8 == 0 &&
        g.bBatch % 8 == 0 && g.aBatch2 % 8 == 0 && g.bBatch2 % 8 == 0) {
      const unsigned tM = (unsigned)((g.M + BM - 1) / BM), tN = (unsigned)((g.N + BN - 1) / BN);
      const LongType tiles = (LongType)tM * tN * batch, KT = (g.K + 63) / 64;
      LongType want = 256 / tiles;             // one round of blocks: a block holds half the LDS of its CU or all of it
      constexpr LongType minPer = 4;   // K-tiles per split at least (the batch-32 decode step: 3 -> 0.556, 4 -> 0.552, 6 -> 0.558, 8 -> 0.555 ms)
      want = want < KT / minPer ? want : KT / minPer;
      want = want < splits ? want : splits;   // the partial-tile scratch bounds chooseSplits' figure
      if (want >= 2) {
        const LongType per = (KT + want - 1) / want;
        g.ktPerSplit = per;
        g.splits = (int)((KT + per - 1) / per);
        constexpr int STAGE_BYTES = (BM + BN) * 8 * 16;
        const bool deep = per > 4 && DynLds<gemm_mfma16s<T, B_KC, 8, 1, true, true, A_KC, true>, 8 * STAGE_BYTES>::granted();
        if (deep || DynLds<gemm_mfma16s<T, B_KC, 4, 1, true, true, A_KC, true>, 4 * STAGE_BYTES>::granted()) {
          noteKernel("gemm_mfma16s<%s,64x64,akc=%d,bkc=%d,stages=%d,split>+splitk_finish", tname<T>(), (int)A_KC, (int)B_KC, deep ? 8 : 4);
          auto kern = deep ? gemm_mfma16s<T, B_KC, 8, 1, true, true, A_KC, true> : gemm_mfma16s<T, B_KC, 4, 1, true, true, A_KC, true>;
          hipLaunchKernelGGL(kern, dim3(tM * tN, (unsigned)g.splits, (unsigned)batch), dim3(256), (deep ? 8 : 4) * STAGE_BYTES, s, g, (const T*)A, (const T*)B,
                             (T*)C, tM, tN);
          hipLaunchKernelGGL((splitk_finish<T, BM, BN, WM, WN>), dim3(tM * tN, (BM / WM / 32) * (BN / WN / 32) * 4, (unsigned)batch), dim3(NT), 0, s, g, (T*)C, tM, tN);
          return true;
        }
        g.splits = splits;   // back to the register-staged split
        LongType per0 = 0;
        chooseSplits<BM, BN>(g, batch, per0);
        g.ktPerSplit = per0;
      }
    }
  }
  const bool usePipe = splits == 1;   // the split-K epilogue lives in the plain kernel
  // whole tiles only: the kernel without bounds handling (its K loop needs two K-tiles at least)
  const bool useFull = aligned && usePipe && BM * BN >= 128 * 128 && g.M % BM == 0 && g.N % BN == 0 && g.K % 64 == 0 && g.K >= 128;
  // small tiles, at most a couple per CU and a long K: the loop is bound by one memory latency per K-tile unless several
  // K-tiles are in flight
  const unsigned nTiles = (unsigned)(((g.M + BM - 1) / BM) * ((g.N + BN - 1) / BN) * batch);
  const bool useDeep = aligned && usePipe && !useFull && BM * BN <= 64 * 64 && nTiles <= 1024 && g.K >= 512 && g.M % BM == 0 && g.N % BN == 0 && g.K % 256 == 0;
  // the direct-load ring takes the small-tile launches it can: 64 x 64 or 128 x 128 tiles, A k-contiguous, 16-byte aligned rows
  if constexpr ((BM == 64 && BN == 64 || BM == 128 && BN == 128) && WM == 2 && WN == 2) {
    constexpr int TW = BM / 64;
    constexpr int STAGE_BYTES = (BM + BN) * 8 * 16;
    static const bool small = getenv("ND4JHIP_GEMM_SMALL_RING") ? atoi(getenv("ND4JHIP_GEMM_SMALL_RING")) != 0 : true;
    const LongType ldaS = A_KC ? g.aRow : g.aCol, ldbS = B_KC ? g.bCol : g.bRow;
    // ragged M / N, or a K that is not a whole number of K-tiles: the edge instantiation, with the zero page for the end of
    // K where K is not a multiple of 256 (whole tiles and a K of whole K-tiles keep the kernels they had)
    const bool ktail = g.K % 256 != 0;
    // from K = 128 on (1000 x 1000 x 136: 7.4 -> 4.7 us, 2000 x 2000 x 456: 19.5 -> 11.4 us against the bounds-handling kernel)
    constexpr LongType edgeMinK = 128;
    const bool edgeShape = (!whole || g.K % 64 != 0) && edge && edgeOk && aligned && usePipe && nTiles <= 1024 && g.K >= edgeMinK;
    const bool shape = edgeShape || (TW == 1 ? useDeep : (useFull && nTiles <= 1024 && g.K >= 512 && g.K % 256 == 0));
    if (small && shape && ldaS % 8 == 0 && ldbS % 8 == 0 && ldaS < (1 << 23) && ldbS < (1 << 23) &&
        ((reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(B)) & 15) == 0 && g.aBatch % 8 == 0 && g.bBatch % 8 == 0 &&
        g.aBatch2 % 8 == 0 && g.bBatch2 % 8 == 0) {
      const unsigned tM = (unsigned)((g.M + BM - 1) / BM), tN = (unsigned)((g.N + BN - 1) / BN);
      // 64 x 64: one tile per CU and a K of whole eight-tile rounds take eight stages (128 KiB), else four (two blocks fit a
      // CU); 128 x 128: four stages (128 KiB)
      constexpr int DEEP = TW == 1 ? 8 : 4;
      // a K that ends inside a round of eight K-tiles multiplies zeros for the rest of it: eight stages only if that is at
      // most one K-tile
      const LongType kTiles = (g.K + 63) / 64;
      const bool wantDeep = TW == 2 || (nTiles <= 256 && (ktail ? (kTiles + 7) / 8 * 8 - kTiles <= 1 : g.K % 512 == 0));
      const bool plain = !edgeShape;
      const bool grantedDeep = plain   ? DynLds<gemm_mfma16s<T, B_KC, DEEP, TW, false, false, A_KC>, DEEP * STAGE_BYTES>::granted()
                               : ktail ? DynLds<gemm_mfma16s<T, B_KC, DEEP, TW, true, true, A_KC>, DEEP * STAGE_BYTES>::granted()
                                       : DynLds<gemm_mfma16s<T, B_KC, DEEP, TW, true, false, A_KC>, DEEP * STAGE_BYTES>::granted();
      const char* const flavour = plain ? "" : ktail ? ",edge,ktail" : ",edge";
      if (wantDeep && grantedDeep) {
        noteKernel("gemm_mfma16s<%s,%dx%d,akc=%d,bkc=%d,stages=%d%s>", tname<T>(), BM, BN, (int)A_KC, (int)B_KC, DEEP, flavour);
        auto kern = plain   ? gemm_mfma16s<T, B_KC, DEEP, TW, false, false, A_KC>
                    : ktail ? gemm_mfma16s<T, B_KC, DEEP, TW, true, true, A_KC> : gemm_mfma16s<T, B_KC, DEEP, TW, true, false, A_KC>;
        hipLaunchKernelGGL(kern, dim3(tM * tN, 1, (unsigned)batch), dim3(256), DEEP * STAGE_BYTES, s, g, (const T*)A, (const T*)B, (T*)C, tM, tN);
        return true;
      }
      if constexpr (TW == 1) {
        noteKernel("gemm_mfma16s<%s,64x64,akc=%d,bkc=%d,stages=4%s>", tname<T>(), (int)A_KC, (int)B_KC, flavour);
        auto kern = plain   ? gemm_mfma16s<T, B_KC, 4, 1, false, false, A_KC>
                    : ktail ? gemm_mfma16s<T, B_KC, 4, 1, true, true, A_KC> : gemm_mfma16s<T, B_KC, 4, 1, true, false, A_KC>;
        hipLaunchKernelGGL(kern, dim3(tM * tN, 1, (unsigned)batch), dim3(256), 4 * STAGE_BYTES, s, g, (const T*)A, (const T*)B, (T*)C, tM, tN);
        return true;
      }
    }
  }
  auto kern = useFull ? gemm_mfma16f<T, BM, BN, WM, WN, A_KC, B_KC>
              : useDeep ? gemm_mfma16q<T, BM, BN, WM, WN, A_KC, B_KC, 4>
              : usePipe ? gemm_mfma16p<T, BM, BN, WM, WN, A_KC, B_KC> : gemm_mfma16<T, BM, BN, WM, WN, A_KC, B_KC>;
  const bool ldsGranted = useFull ? DynLds<gemm_mfma16f<T, BM, BN, WM, WN, A_KC, B_KC>, (int)LDS>::granted()
                          : useDeep ? DynLds<gemm_mfma16q<T, BM, BN, WM, WN, A_KC, B_KC, 4>, (int)LDS>::granted()
                          : usePipe ? DynLds<gemm_mfma16p<T, BM, BN, WM, WN, A_KC, B_KC>, (int)LDS>::granted()
                                    : DynLds<gemm_mfma16<T, BM, BN, WM, WN, A_KC, B_KC>, (int)LDS>::granted();
  ND4J_REQUIRE(ldsGranted, "matmul: the device does not grant the tile kernel its LDS");
  const unsigned tilesM = (unsigned)((g.M + BM - 1) / BM), tilesN = (unsigned)((g.N + BN - 1) / BN);
  if constexpr (BM == 32) {
    // a few rows against a matrix that is large against the last-level cache (the logits of a decode step against the
    // embedding: 77 MB): every element of B is read once, through non-temporal loads, and what the step reads again -- the
    // layers' weights -- stays in the cache (batch-32 step 0.616 -> see the bench line)
    if (usePipe && !useFull && !useDeep && tilesM == 1 && batch == 1 &&
        (double)g.N * (double)g.K * sizeof(T) >= (double)(32 << 20) &&
        DynLds<gemm_mfma16p<T, BM, BN, WM, WN, A_KC, B_KC, true>, (int)LDS>::granted())
      kern = gemm_mfma16p<T, BM, BN, WM, WN, A_KC, B_KC, true>;
  }
  noteKernel("%s<%s,%dx%d,akc=%d,bkc=%d>%s", useFull ? "gemm_mfma16f" : useDeep ? "gemm_mfma16q" : usePipe ? "gemm_mfma16p" : "gemm_mfma16", tname<T>(), BM, BN,
             (int)A_KC, (int)B_KC, splits > 1 ? "+splitk_finish" : "");
  hipLaunchKernelGGL(kern, dim3(tilesM * tilesN, (unsigned)splits, (unsigned)batch), dim3(NT), LDS, s, g, (const T*)A, (const T*)B, (T*)C, tilesM, tilesN);
  if (splits > 1)
    hipLaunchKernelGGL((splitk_finish<T, BM, BN, WM, WN>), dim3(tilesM * tilesN, (BM / WM / 32) * (BN / WN / 32) * 4, (unsigned)batch), dim3(NT), 0, s, g, (T*)C, tilesM, tilesN);
  return true;
}

template <typename T, bool A_KC, bool B_KC>
static bool launchMfma16(hipStream_t s, const GemmArgs& g, const void* A, const void* B, void* C, LongType batch, bool aligned) {
  const LongType tiles256 = ((g.M + 255) / 256) * ((g.N + 255) / 256) * batch;
  const LongType tiles128 = ((g.M + 127) / 128) * ((g.N + 127) / 128) * batch;
  // up to 32 rows against a long K (a batched decode step's second MLP product, K = 3072): the 64 x 64 configuration, whose
  // split-K runs on the direct-load ring (7.6 against 8.7 us with the 32 x 128 tiles of the register-staged split)
  static const bool skinnyRing = getenv("ND4JHIP_GEMM_SKINNY_RING") ? atoi(getenv("ND4JHIP_GEMM_SKINNY_RING")) != 0 : true;
  if (g.M <= 32 && skinnyRing && aligned && g.K >= 2048 && launchMfma16Cfg<T, 64, 64, 2, 2, A_KC, B_KC>(s, g, A, B, C, batch, true, aligned)) return true;
  if (g.M <= 32) return launchMfma16Cfg<T, 32, 128, 1, 4, A_KC, B_KC>(s, g, A, B, C, batch, true, aligned);
  if (g.M <= 64 || g.N <= 64 || tiles128 < 192) return launchMfma16Cfg<T, 64, 64, 2, 2, A_KC, B_KC>(s, g, A, B, C, batch, true, aligned);
  if (tiles256 < 192) return launchMfma16Cfg<T, 128, 128, 2, 2, A_KC, B_KC>(s, g, A, B, C, batch, false, aligned);
  if (g.hasEpi) return false;
  if constexpr (!A_KC && !B_KC) {
    // the same for a transposed A (the two-stage kernel with both operands' k-rows in LDS as they lie in memory)
    static const bool ub = getenv("ND4JHIP_GEMM_UNALIGNED_RING") ? atoi(getenv("ND4JHIP_GEMM_UNALIGNED_RING")) != 0 : true;
    constexpr size_t LDS = 2 * 2 * 256 * 8 * 16;
    if (!aligned && ub && batch == 1 && (reinterpret_cast<uintptr_t>(A) & 15) == 0 && g.aCol % 8 == 0 && g.M % 8 == 0 && g.K >= 128 && g.N >= 264 &&
        DynLds<gemm_mfma16d<T, false, true, false, false>, (int)LDS>::granted() && DynLds<gemm_mfma16d<T, false, true, true, false>, (int)LDS>::granted()) {
      GemmArgs g1 = g;
      g1.N = g.N & ~(LongType)7;
      const unsigned tM = (unsigned)((g.M + 255) / 256), tN = (unsigned)((g1.N + 255) / 256);
      auto kern = g.K % 64 == 0 ? gemm_mfma16d<T, false, true, false, false> : gemm_mfma16d<T, false, true, true, false>;
      hipLaunchKernelGGL(kern, dim3(tM * tN, 1, 1), dim3(512), LDS, s, g1, (const T*)A, (const T*)B, (T*)C, tM, tN);
      const LongType rem = g.N & 7;
      if (rem) {
        GemmArgs g2 = g;
        g2.N = rem;
        if (g.bias) g2.bias = static_cast<const T*>(g.bias) + g1.N;
        if (!launchMfma16Cfg<T, 64, 64, 2, 2, A_KC, B_KC>(s, g2, A, (const T*)B + g1.N, (T*)C + g1.N * g.cCol, 1, false, false)) return false;
      }
      noteKernel("gemm_mfma16d<%s,256x256,akc=0,bkc=0,edge%s,unaligned>", tname<T>(), g.K % 64 == 0 ? "" : ",ktail");
      return true;
    }
  }
  if constexpr (A_KC && !B_KC) {
    // A row-major B whose rows start off 16-byte boundaries (a [768, 50257] matrix) with everything else in place for the
    // ring kernel: its loads into LDS take element-aligned addresses like any other global load, and every column group
    // of 8 is whole up to the last multiple of 8 -- the edge instantiation over those columns, then the up to 7 columns
    // that are left through the bounds-handling kernel (bf16 4096 x 50257 x 768: 0.71 -> 0.40 ms)
    static const bool ub = getenv("ND4JHIP_GEMM_UNALIGNED_RING") ? atoi(getenv("ND4JHIP_GEMM_UNALIGNED_RING")) != 0 : true;
    constexpr size_t LDS = (3 * 256 * 8 + 4 * 32 * 32) * 16;
    if (!aligned && ub && batch == 1 && (reinterpret_cast<uintptr_t>(A) & 15) == 0 && g.aRow % 8 == 0 && g.K % 8 == 0 && g.K >= 128 && g.N >= 264 &&
        DynLds<gemm_mfma16r<T, true>, (int)LDS>::granted() && DynLds<gemm_mfma16r<T, true, true>, (int)LDS>::granted()) {
      GemmArgs g1 = g;
      g1.N = g.N & ~(LongType)7;
      const unsigned tM = (unsigned)((g.M + 255) / 256), tN = (unsigned)((g1.N + 255) / 256);
      auto kern = g.K % 128 == 0 ? gemm_mfma16r<T, true, false> : gemm_mfma16r<T, true, true>;
      hipLaunchKernelGGL(kern, dim3(tM * tN, 1, 1), dim3(512), LDS, s, g1, (const T*)A, (const T*)B, (T*)C, tM, tN);
      const LongType rem = g.N & 7;
      if (rem) {
        GemmArgs g2 = g;
        g2.N = rem;
        if (g.bias) g2.bias = static_cast<const T*>(g.bias) + g1.N;
        if (!launchMfma16Cfg<T, 64, 64, 2, 2, A_KC, B_KC>(s, g2, A, (const T*)B + g1.N, (T*)C + g1.N * g.cCol, 1, false, false)) return false;
      }
      noteKernel("gemm_mfma16r<%s,256x256,akc=1,bkc=0,edge%s,unaligned>", tname<T>(), g.K % 128 == 0 ? "" : ",ktail");
      return true;
    }
  }
  if (!aligned) return launchMfma16Cfg<T, 256, 256, 2, 4, A_KC, B_KC>(s, g, A, B, C, batch, false, false);
  static const bool direct = getenv("ND4JHIP_GEMM_DIRECT") ? atoi(getenv("ND4JHIP_GEMM_DIRECT")) != 0 : true;
  static const bool ring = getenv("ND4JHIP_GEMM_RING") ? atoi(getenv("ND4JHIP_GEMM_RING")) != 0 : true;
  // the direct-load kernels take an M or N that is not a whole number of tiles through their edge instantiations (a
  // row-major B in whole 16-byte column groups only)
  static const bool edge = getenv("ND4JHIP_GEMM_EDGE") ? atoi(getenv("ND4JHIP_GEMM_EDGE")) != 0 : true;
  const bool whole = g.M % 256 == 0 && g.N % 256 == 0;
  const bool edgeOk = whole || (edge && (B_KC || g.N % 8 == 0) && (A_KC || g.M % 8 == 0));
  const unsigned tM = (unsigned)((g.M + 255) / 256), tN = (unsigned)((g.N + 255) / 256);
  if constexpr (A_KC && !B_KC) {
    constexpr size_t LDS = (3 * 256 * 8 + 4 * 32 * 32) * 16;   // 160 KiB: the whole LDS of a CU
    // a device or driver that does not grant a block the whole LDS keeps the two-stage kernel below
    const bool ringGranted = whole ? DynLds<gemm_mfma16r<T>, (int)LDS>::granted() : DynLds<gemm_mfma16r<T, true>, (int)LDS>::granted();
    if (direct && ring && ringGranted && edgeOk && g.K % 128 == 0) {
      noteKernel("gemm_mfma16r<%s,256x256,akc=1,bkc=0%s>", tname<T>(), whole ? "" : ",edge");
      auto kern = whole ? gemm_mfma16r<T, false> : gemm_mfma16r<T, true>;
      hipLaunchKernelGGL(kern, dim3(tM * tN, 1, (unsigned)batch), dim3(512), LDS, s, g, (const T*)A, (const T*)B, (T*)C, tM, tN);
      return true;
    }
    // a K that is not a whole number of K-tiles: the ring over K rounded up, zeros from K on (a K of whole 64-k tiles keeps
    // the two-stage kernel below)
    if (direct && ring && edge && edgeOk && g.K % 64 != 0 && g.K >= 128 && DynLds<gemm_mfma16r<T, true, true>, (int)LDS>::granted()) {
      noteKernel("gemm_mfma16r<%s,256x256,akc=1,bkc=0,edge,ktail>", tname<T>());
      auto kern = gemm_mfma16r<T, true, true>;
      hipLaunchKernelGGL(kern, dim3(tM * tN, 1, (unsigned)batch), dim3(512), LDS, s, g, (const T*)A, (const T*)B, (T*)C, tM, tN);
      return true;
    }
  }
  if (direct && A_KC && edgeOk && g.K % 64 == 0 && g.K >= 128) {
    constexpr size_t LDS = 2 * 2 * 256 * 8 * 16;
    const bool granted = whole ? DynLds<gemm_mfma16d<T, B_KC>, (int)LDS>::granted() : DynLds<gemm_mfma16d<T, B_KC, true>, (int)LDS>::granted();
    ND4J_REQUIRE(granted, "matmul: the device does not grant the two-stage kernel its LDS");
    noteKernel("gemm_mfma16d<%s,256x256,akc=1,bkc=%d%s>", tname<T>(), (int)B_KC, whole ? "" : ",edge");
    auto kern = whole ? gemm_mfma16d<T, B_KC, false> : gemm_mfma16d<T, B_KC, true>;
    hipLaunchKernelGGL(kern, dim3(tM * tN, 1, (unsigned)batch), dim3(512), LDS, s, g, (const T*)A, (const T*)B, (T*)C, tM, tN);
    return true;
  }
  if constexpr (A_KC && B_KC) {
    constexpr size_t LDS = 2 * 2 * 256 * 8 * 16;
    if (direct && edge && edgeOk && g.K % 64 != 0 && g.K >= 128 && DynLds<gemm_mfma16d<T, true, true, true>, (int)LDS>::granted()) {
      noteKernel("gemm_mfma16d<%s,256x256,akc=1,bkc=1,edge,ktail>", tname<T>());
      auto kern = gemm_mfma16d<T, true, true, true>;
      hipLaunchKernelGGL(kern, dim3(tM * tN, 1, (unsigned)batch), dim3(512), LDS, s, g, (const T*)A, (const T*)B, (T*)C, tM, tN);
      return true;
    }
  }
  if constexpr (!A_KC) {
    // a transposed A: the two-stage direct-load kernel with A's k-rows in LDS as they lie in memory
    static const bool taDirect = getenv("ND4JHIP_GEMM_TA_DIRECT") ? atoi(getenv("ND4JHIP_GEMM_TA_DIRECT")) != 0 : true;
    constexpr size_t LDS = 2 * 2 * 256 * 8 * 16;
    const bool ktail = g.K % 64 != 0;
    if (direct && taDirect && edgeOk && g.K >= 128 && (edge || (whole && !ktail))) {
      auto kern = ktail   ? gemm_mfma16d<T, B_KC, true, true, false>
                  : whole ? gemm_mfma16d<T, B_KC, false, false, false> : gemm_mfma16d<T, B_KC, true, false, false>;
      const bool granted = ktail   ? DynLds<gemm_mfma16d<T, B_KC, true, true, false>, (int)LDS>::granted()
                           : whole ? DynLds<gemm_mfma16d<T, B_KC, false, false, false>, (int)LDS>::granted()
                                   : DynLds<gemm_mfma16d<T, B_KC, true, false, false>, (int)LDS>::granted();
      if (granted) {
        noteKernel("gemm_mfma16d<%s,256x256,akc=0,bkc=%d%s>", tname<T>(), (int)B_KC, ktail ? ",edge,ktail" : whole ? "" : ",edge");
        hipLaunchKernelGGL(kern, dim3(tM * tN, 1, (unsigned)batch), dim3(512), LDS, s, g, (const T*)A, (const T*)B, (T*)C, tM, tN);
        return true;
      }
    }
  }
  return launchMfma16Cfg<T, 256, 256, 2, 4, A_KC, B_KC>(s, g, A, B, C, batch, false, true);
}

// ---- fp32 MFMA kernel ------------------------------------------------------------------------------------------------
// tile BM x BN x 16; LDS holds [k][row + pad] floats; one MFMA 32x32x2 consumes k = 2*s + lane/32, row = lane%32
template <int BM, int BN, int WM, int WN, bool A_KC, bool B_KC>
__global__ __launch_bounds__(WM * WN * 64) void gemm_mfma32(GemmArgs g, const float* __restrict__ A, const float* __restrict__ B,
                                                             float* __restrict__ C, unsigned tilesM, unsigned tilesN) {
  constexpr int BK = 16, NT = WM * WN * 64, PA = BM + 4, PB = BN + 4;
  constexpr int WTM = BM / WM, WTN = BN / WN, TM = WTM / 32, TN = WTN / 32;
  constexpr int VA = BM * BK / 4 / NT, VB = BN * BK / 4 / NT;   // float4 per thread
  __shared__ __attribute__((aligned(16))) float sA[2][BK * PA];
  __shared__ __attribute__((aligned(16))) float sB[2][BK * PB];
  unsigned tm, tn;
  tileOf(blockIdx.x, gridDim.x, tilesM, tilesN, tm, tn);
  const LongType m0 = (LongType)tm * BM, n0 = (LongType)tn * BN;
  const LongType bz = blockIdx.z;
  { LongType oa, ob, oc; batchOffsets(g, bz, oa, ob, oc); A += oa; B += ob; C += oc; }
  const LongType lda = A_KC ? g.aRow : g.aCol, ldb = B_KC ? g.bCol : g.bRow;
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6, wm = wave / WN, wn = wave % WN;
  typedef __attribute__((ext_vector_type(4))) float f32x4;
  f32x16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int j = 0; j < TN; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;
  f32x4 ra[VA], rb[VB];
  const f32x4 zero = {0.f, 0.f, 0.f, 0.f};

  // Rows need element alignment only and the contiguous extent need not be a multiple of 4: every load is an unconditional
  // 16-byte read from a position inside the operand (a group that would run over the end of its row is read 4 elements back
  // from the end and moved down in registers, zeros coming in; k positions past K give zeros; rows past the limit of a
  // k-contiguous operand repeat the last row).  Needs K >= 4 (k-contiguous) or 4 rows (row-contiguous).
  auto vec4 = [&](const float* p) { f32x4 v; __builtin_memcpy(&v, p, 16); return v; };
  auto down = [&](f32x4 v, int sh) {
    f32x4 o;
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const int i = j + sh;
      o[j] = i == 0 ? v[0] : i == 1 ? v[1] : i == 2 ? v[2] : i == 3 ? v[3] : 0.f;
    }
    return o;
  };
  auto loadTile = [&](auto& reg, auto nv, auto kc, auto rows, const float* base, LongType ld, LongType row0, LongType limit, LongType k0) {
    constexpr int NV = decltype(nv)::value, ROWS = decltype(rows)::value;
    constexpr bool KC = decltype(kc)::value;
#pragma unroll
    for (int i = 0; i < NV; i++) {
      const int v = t + i * NT;
      if (KC) {
        const int kq = v & 3, row = v >> 2;
        LongType r = row0 + row; r = r < limit ? r : limit - 1;
        const LongType k = k0 + kq * 4, kk = k + 4 <= g.K ? k : g.K - 4;
        reg[i] = vec4(base + r * ld + kk);
        if (k != kk) reg[i] = down(reg[i], (int)(k - kk < 4 ? k - kk : 4));
      } else {
        const int rq = v % (ROWS / 4), kk = v / (ROWS / 4);
        const LongType r = row0 + rq * 4, rr = r + 4 <= limit ? r : limit - 4;
        const LongType k = k0 + kk;
        reg[i] = vec4(base + (k < g.K ? k : g.K - 1) * ld + rr);
        if (k >= g.K) reg[i] = zero;
        else if (r != rr) reg[i] = down(reg[i], (int)(r - rr < 4 ? r - rr : 4));
      }
    }
  };
  auto loadA = [&](LongType k0) {
    loadTile(ra, std::integral_constant<int, VA>(), std::integral_constant<bool, A_KC>(), std::integral_constant<int, BM>(), A, lda, m0, g.M, k0);
  };
  auto loadB = [&](LongType k0) {
    loadTile(rb, std::integral_constant<int, VB>(), std::integral_constant<bool, B_KC>(), std::integral_constant<int, BN>(), B, ldb, n0, g.N, k0);
  };
  auto storeA = [&](int stage) {
#pragma unroll
    for (int i = 0; i < VA; i++) {
      const int v = t + i * NT;
      if (A_KC) {
        const int kq = v & 3, row = v >> 2;
#pragma unroll
        for (int q = 0; q < 4; q++) sA[stage][(kq * 4 + q) * PA + row] = ra[i][q];
      } else {
        const int rq = v % (BM / 4), kk = v / (BM / 4);
        *reinterpret_cast<f32x4*>(&sA[stage][kk * PA + rq * 4]) = ra[i];
      }
    }
  };
  auto storeB = [&](int stage) {
#pragma unroll
    for (int i = 0; i < VB; i++) {
      const int v = t + i * NT;
      if (B_KC) {
        const int kq = v & 3, row = v >> 2;
#pragma unroll
        for (int q = 0; q < 4; q++) sB[stage][(kq * 4 + q) * PB + row] = rb[i][q];
      } else {
        const int rq = v % (BN / 4), kk = v / (BN / 4);
        *reinterpret_cast<f32x4*>(&sB[stage][kk * PB + rq * 4]) = rb[i];
      }
    }
  };

  const LongType KT = (g.K + BK - 1) / BK;
  loadA(0); loadB(0); storeA(0); storeB(0);
  __syncthreads();
  for (LongType kt = 0; kt < KT; kt++) {
    const int cur = (int)(kt & 1);
    if (kt + 1 < KT) { loadA((kt + 1) * BK); loadB((kt + 1) * BK); }
#pragma unroll
    for (int ks = 0; ks < BK / 2; ks++) {
      const int k = ks * 2 + (lane >> 5);
      float fa[TM], fb[TN];
#pragma unroll
      for (int i = 0; i < TM; i++) fa[i] = sA[cur][k * PA + wm * WTM + i * 32 + (lane & 31)];
#pragma unroll
      for (int j = 0; j < TN; j++) fb[j] = sB[cur][k * PB + wn * WTN + j * 32 + (lane & 31)];
#pragma unroll
      for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i], fb[j], acc[i][j], 0, 0, 0);
    }
    if (kt + 1 < KT) { storeA(cur ^ 1); storeB(cur ^ 1); }
    __syncthreads();
  }
  storeAccTiles<float, TM, TN, true>(g, C, acc, m0 + wm * WTM, n0 + wn * WTN, lane);
}

// The fp32 kernel for launches of whole tiles that put one small tile on a CU: PD K-tiles of global loads in flight (PD
// register sets, the K loop unrolled PD times and free of branches -- loads past the end re-read the last K-tile, the
// store after the last K-tile fills a stage nobody reads), so the loop runs at the MFMA rate instead of one memory
// latency per K-tile.  BK = 32 halves the barriers per MFMA (the one-tile-per-CU launch, where nothing else covers
// them).  Host: K % (BK * PD) == 0, K >= 2 * BK * PD; M % BM == 0 and N % BN == 0 unless EDGE: then the rows (the 16-byte
// groups along M or N of an operand that is contiguous that way) beyond the edge are read from clamped positions inside the
// operand and only reach elements of C that the bounds-checked store leaves out.
// KTAIL: K need not be a whole number of rounds (a multiple of 4 where an operand is k-contiguous) -- the loop runs over K
// rounded up to PD K-tiles and a lane whose 16 bytes start at k >= K reads a page of zeros.
template <int BM, int BN, int WM, int WN, bool A_KC, bool B_KC, int PD, int BK, bool EDGE = false, bool KTAIL = false>
__global__ __launch_bounds__(WM * WN * 64) void gemm_mfma32q(GemmArgs g, const float* __restrict__ A, const float* __restrict__ B,
                                                              float* __restrict__ C, unsigned tilesM, unsigned tilesN) {
  static_assert(PD % 2 == 0, "the LDS stage of a K-tile must be a compile-time constant inside the unrolled loop");
  static_assert(BK == 16 || BK == 32, "K-tile");
  // row pitch of a stage: k-contiguous operands are scattered into it (a thread's 4 k land 4 rows apart, KQ threads share a
  // row of the operand): 4 * pitch mod 64 banks must be 64 / KQ apart; the others are stored 16 bytes at a time
  constexpr int KQ = BK / 4, NT = WM * WN * 64, PA = BM + (A_KC && BK == 32 ? 2 : 4), PB = BN + (B_KC && BK == 32 ? 2 : 4);
  constexpr int WTM = BM / WM, WTN = BN / WN, TM = WTM / 32, TN = WTN / 32;
  constexpr int VA = BM * BK / 4 / NT, VB = BN * BK / 4 / NT;   // float4 per thread
  __shared__ __attribute__((aligned(16))) float sA[2][BK * PA];
  __shared__ __attribute__((aligned(16))) float sB[2][BK * PB];
  unsigned tm, tn;
  tileOf(blockIdx.x, gridDim.x, tilesM, tilesN, tm, tn);
  const LongType m0 = (LongType)tm * BM, n0 = (LongType)tn * BN;
  const LongType bz = blockIdx.z;
  { LongType oa, ob, oc; batchOffsets(g, bz, oa, ob, oc); A += oa; B += ob; C += oc; }
  const LongType lda = A_KC ? g.aRow : g.aCol, ldb = B_KC ? g.bCol : g.bRow;
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6, wm = wave / WN, wn = wave % WN;
  typedef __attribute__((ext_vector_type(4))) float f32x4;
  f32x16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int j = 0; j < TN; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;
  f32x4 ra[PD][VA], rb[PD][VB];
  // Every thread keeps one running pointer per load, advanced by the K-tile's byte step (the same for all lanes: a scalar
  // operand, set to zero once the last K-tile is reached so that loads past the end re-read it): one 64-bit add per load
  // and K-tile.  Computed from the element coordinates each time it cost a 64-bit multiply-add chain in front of an MFMA.
  typedef const __attribute__((address_space(1))) char* GlobalBytes;
  GlobalBytes curA[VA], curB[VB];
  int kOffA[VA], kOffB[VB];   // KTAIL: the k (inside a K-tile) this lane's 16 bytes start at
#pragma unroll
  for (int i = 0; i < VA; i++) kOffA[i] = A_KC ? ((t + i * NT) % KQ) * 4 : (t + i * NT) / (BM / 4);
#pragma unroll
  for (int i = 0; i < VB; i++) kOffB[i] = B_KC ? ((t + i * NT) % KQ) * 4 : (t + i * NT) / (BN / 4);
#pragma unroll
  for (int i = 0; i < VA; i++) {
    const int v = t + i * NT;
    LongType am = A_KC ? m0 + v / KQ : m0 + (v % (BM / 4)) * 4;
    if (EDGE) am = A_KC ? (am < g.M ? am : g.M - 1) : (am + 4 <= g.M ? am : g.M - 4);
    curA[i] = (GlobalBytes)(A_KC ? A + am * lda + (v % KQ) * 4 : A + (LongType)(v / (BM / 4)) * lda + am);
  }
#pragma unroll
  for (int i = 0; i < VB; i++) {
    const int v = t + i * NT;
    LongType bn = B_KC ? n0 + v / KQ : n0 + (v % (BN / 4)) * 4;
    if (EDGE) bn = B_KC ? (bn < g.N ? bn : g.N - 1) : (bn + 4 <= g.N ? bn : g.N - 4);
    curB[i] = (GlobalBytes)(B_KC ? B + bn * ldb + (v % KQ) * 4 : B + (LongType)(v / (BN / 4)) * ldb + bn);
  }
  const LongType KT = KTAIL ? (g.K + BK * PD - 1) / (BK * PD) * PD : g.K / BK;
  const LongType stepA = (A_KC ? BK : BK * lda) * 4, stepB = (B_KC ? BK : BK * ldb) * 4;   // bytes per K-tile
  int kNext = 0;   // KTAIL: first k of the K-tile the pointers stand at (they move on with every load there)
  const GlobalBytes zero = (GlobalBytes)gemmZeroPage;
  // more: the K-tile loaded is not the last one (a condition on the loop counters, so a scalar one)
  auto loadNext = [&](int u, bool more) {
#pragma unroll
    for (int i = 0; i < VA; i++) ra[u][i] = *(const __attribute__((address_space(1))) f32x4*)(!KTAIL || kNext + kOffA[i] < (int)g.K ? curA[i] : zero);
#pragma unroll
    for (int i = 0; i < VB; i++) rb[u][i] = *(const __attribute__((address_space(1))) f32x4*)(!KTAIL || kNext + kOffB[i] < (int)g.K ? curB[i] : zero);
    if (KTAIL) { more = true; kNext += BK; }
    const LongType sa = more ? stepA : 0, sb = more ? stepB : 0;
#pragma unroll
    for (int i = 0; i < VA; i++) curA[i] += sa;
#pragma unroll
    for (int i = 0; i < VB; i++) curB[i] += sb;
  };
  auto storeA = [&](int u, int stage, int i) {
    const int v = t + i * NT;
    if (A_KC) {
#pragma unroll
      for (int q = 0; q < 4; q++) sA[stage][((v % KQ) * 4 + q) * PA + v / KQ] = ra[u][i][q];
    } else {
      *reinterpret_cast<f32x4*>(&sA[stage][(v / (BM / 4)) * PA + (v % (BM / 4)) * 4]) = ra[u][i];
    }
  };
  auto storeB = [&](int u, int stage, int i) {
    const int v = t + i * NT;
    if (B_KC) {
#pragma unroll
      for (int q = 0; q < 4; q++) sB[stage][((v % KQ) * 4 + q) * PB + v / KQ] = rb[u][i][q];
    } else {
      *reinterpret_cast<f32x4*>(&sB[stage][(v / (BN / 4)) * PB + (v % (BN / 4)) * 4]) = rb[u][i];
    }
  };
  auto store = [&](int u, int stage) {
#pragma unroll
    for (int i = 0; i < VA; i++) storeA(u, stage, i);
#pragma unroll
    for (int i = 0; i < VB; i++) storeB(u, stage, i);
  };
#pragma unroll
  for (int u = 0; u < PD; u++) loadNext(u, true);   // KT >= 2 * PD
  store(0, 0);
  __syncthreads();
  // One small tile per CU (one wave per SIMD, one accumulator per wave): nothing covers an LDS round trip, so the
  // fragments of K-tile kt + 1 are read right after the barrier that completes its stage, under the MFMAs of K-tile kt
  // (the same arrangement as gemm_mfma16q).  The larger tile keeps the plain order, which is already MFMA-bound.
  constexpr bool EARLY = TM * TN == 1;
  if constexpr (EARLY) {
    float fa[2][BK / 2][TM], fb[2][BK / 2][TN];
    f32x16 acc2[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
      for (int j = 0; j < TN; j++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc2[i][j][r] = 0.f;
    auto readPart = [&](int stage, int buf, int from, int to) {
#pragma unroll
      for (int ks = from; ks < to; ks++) {
        const int k = ks * 2 + (lane >> 5);
#pragma unroll
        for (int i = 0; i < TM; i++) fa[buf][ks][i] = sA[stage][k * PA + wm * WTM + i * 32 + (lane & 31)];
#pragma unroll
        for (int j = 0; j < TN; j++) fb[buf][ks][j] = sB[stage][k * PB + wn * WTN + j * 32 + (lane & 31)];
      }
    };
    constexpr int NS = BK / 2;   // MFMAs (k-steps of 2) per K-tile and accumulator tile
    static_assert(VA + VB + 1 <= NS / 2, "stores and loads go in front of the barrier, one per MFMA");
    readPart(0, 0, 0, NS);
    for (LongType kt0 = 0; kt0 < KT; kt0 += PD) {
#pragma unroll
      for (int u = 0; u < PD; u++) {
        const int cur = u & 1;
        // The wave's own bookkeeping for K-tile kt + 1 is issued between the MFMAs of K-tile kt (64 cycles of matrix pipe
        // each), one piece per MFMA: left in front of them it ran while the pipe stood still, 200 cycles for every 512 of
        // MFMA, and bunched behind one MFMA it overran that MFMA's shadow.  Even and odd k-steps go to two accumulators:
        // with a single one every MFMA would wait for the previous one's result.
#pragma unroll
        for (int ks = 0; ks < NS; ks++) {
#pragma unroll
          for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++) {
              if (ks & 1) acc2[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[cur][ks][i], fb[cur][ks][j], acc2[i][j], 0, 0, 0);
              else acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[cur][ks][i], fb[cur][ks][j], acc[i][j], 0, 0, 0);
            }
          if (ks < VA) storeA((u + 1) % PD, cur ^ 1, ks);
          else if (ks < VA + VB) storeB((u + 1) % PD, cur ^ 1, ks - VA);
          else if (ks == VA + VB) loadNext(u, kt0 + u + PD < KT - 1);   // K-tile min(kt0 + u + PD, KT - 1)
          if (ks == NS / 2 - 1) {
            __builtin_amdgcn_sched_barrier(0);
            __syncthreads();
          }
          if (ks >= NS / 2 && (ks - NS / 2) * 4 < NS) readPart(cur ^ 1, cur ^ 1, (ks - NS / 2) * 4, (ks - NS / 2) * 4 + 4);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
      for (int j = 0; j < TN; j++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[i][j][r] += acc2[i][j][r];
    if (EDGE && (m0 + BM > g.M || n0 + BN > g.N)) storeAccTiles<float, TM, TN, true>(g, C, acc, m0 + wm * WTM, n0 + wn * WTN, lane);
    else storeAccTiles<float, TM, TN, false>(g, C, acc, m0 + wm * WTM, n0 + wn * WTN, lane);
    return;
  }
  for (LongType kt0 = 0; kt0 < KT; kt0 += PD) {
#pragma unroll
    for (int u = 0; u < PD; u++) {
      const int cur = u & 1;
      loadNext(u, kt0 + u + PD < KT - 1);   // K-tile kt0 + u sits in LDS: its register set takes K-tile min(kt0 + u + PD, KT - 1)
#pragma unroll
      for (int ks = 0; ks < BK / 2; ks++) {
        const int k = ks * 2 + (lane >> 5);
        float fa[TM], fb[TN];
#pragma unroll
        for (int i = 0; i < TM; i++) fa[i] = sA[cur][k * PA + wm * WTM + i * 32 + (lane & 31)];
#pragma unroll
        for (int j = 0; j < TN; j++) fb[j] = sB[cur][k * PB + wn * WTN + j * 32 + (lane & 31)];
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
          for (int j = 0; j < TN; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i], fb[j], acc[i][j], 0, 0, 0);
      }
      store((u + 1) % PD, cur ^ 1);
      __syncthreads();
    }
  }
  if (EDGE && (m0 + BM > g.M || n0 + BN > g.N)) storeAccTiles<float, TM, TN, true>(g, C, acc, m0 + wm * WTM, n0 + wn * WTN, lane);
  else storeAccTiles<float, TM, TN, false>(g, C, acc, m0 + wm * WTM, n0 + wn * WTN, lane);
}

template <int BM, int BN, int WM, int WN, bool A_KC, bool B_KC>
static void launchMfma32Cfg(hipStream_t s, const GemmArgs& g, const void* A, const void* B, void* C, LongType batch, bool aligned) {
  const unsigned tilesM = (unsigned)((g.M + BM - 1) / BM), tilesN = (unsigned)((g.N + BN - 1) / BN);
  static const bool edge = getenv("ND4JHIP_GEMM_EDGE") ? atoi(getenv("ND4JHIP_GEMM_EDGE")) != 0 : true;
  const bool whole = g.M % BM == 0 && g.N % BN == 0;
  // `aligned` says that an operand which is contiguous along M or N has an extent of whole 16-byte groups
  const bool ktail = g.K % 128 != 0;
  if (aligned && g.K >= 256 && (whole || (edge && g.M >= 4 && g.N >= 4)) && (!ktail || edge)) {
    constexpr int PD = 4, BK = BM * BN <= 64 * 64 ? 32 : 16;
    noteKernel("gemm_mfma32q<f32,%dx%d,akc=%d,bkc=%d,pd=%d,bk=%d%s>", BM, BN, (int)A_KC, (int)B_KC, PD, BK, ktail ? ",edge,ktail" : whole ? "" : ",edge");
    auto kern = ktail   ? gemm_mfma32q<BM, BN, WM, WN, A_KC, B_KC, PD, BK, true, true>
                : whole ? gemm_mfma32q<BM, BN, WM, WN, A_KC, B_KC, PD, BK, false, false> : gemm_mfma32q<BM, BN, WM, WN, A_KC, B_KC, PD, BK, true, false>;
    hipLaunchKernelGGL(kern, dim3(tilesM * tilesN, 1, (unsigned)batch), dim3(WM * WN * 64), 0, s, g, (const float*)A, (const float*)B, (float*)C,
                       tilesM, tilesN);
    return;
  }
  noteKernel("gemm_mfma32<f32,%dx%d,akc=%d,bkc=%d>", BM, BN, (int)A_KC, (int)B_KC);
  hipLaunchKernelGGL((gemm_mfma32<BM, BN, WM, WN, A_KC, B_KC>), dim3(tilesM * tilesN, 1, (unsigned)batch), dim3(WM * WN * 64), 0, s, g,
                     (const float*)A, (const float*)B, (float*)C, tilesM, tilesN);
}
template <bool A_KC, bool B_KC>
static void launchMfma32(hipStream_t s, const GemmArgs& g, const void* A, const void* B, void* C, LongType batch, bool aligned) {
  const LongType tiles128 = ((g.M + 127) / 128) * ((g.N + 127) / 128) * batch;
  if (g.M <= 64 || g.N <= 64 || tiles128 < 192) return launchMfma32Cfg<64, 64, 2, 2, A_KC, B_KC>(s, g, A, B, C, batch, aligned);
  return launchMfma32Cfg<128, 128, 2, 2, A_KC, B_KC>(s, g, A, B, C, batch, aligned);
}

// ---- GEMV: one skinny operand, the matrix is streamed once ----------------------------------------------------------
// y[n] = alpha * sum_k x[k] * W[n][k] (+ beta y): W rows contiguous in k.  One wave per output row.
template <typename T>
__global__ __launch_bounds__(256) void gemv_rowdot(const T* __restrict__ W, LongType ldw, const T* __restrict__ x, LongType xs, T* __restrict__ y,
                                                   LongType ys, LongType N, LongType K, float alpha, float beta, const T* __restrict__ bias) {
  using A = typename Conv<T>::acc;
  constexpr int V = 16 / sizeof(T);
  using VT = Vec<T, V>;
  const int lane = threadIdx.x & 63;
  const LongType n = (LongType)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (n >= N) return;
  const T* w = W + n * ldw;
  A acc = 0;
  const bool vec = xs == 1 && K % V == 0 && ((reinterpret_cast<uintptr_t>(w) | reinterpret_cast<uintptr_t>(x)) & 15) == 0;
  if (vec) {
    const VT* wv = reinterpret_cast<const VT*>(w);
    const VT* xv = reinterpret_cast<const VT*>(x);
    for (LongType i = lane; i < K / V; i += 64) {
      VT a = wv[i], b = xv[i];
#pragma unroll
      for (int e = 0; e < V; e++) acc += (A)to_float(a.v[e]) * (A)to_float(b.v[e]);
    }
  } else {
    for (LongType k = lane; k < K; k += 64) acc += (A)to_float(w[k]) * (A)to_float(x[k * xs]);
  }
  acc = wave_allreduce<SumOp>(acc);
  if (lane == 0) {
    A v = (A)alpha * acc;
    if (beta != 0.f) v += (A)beta * (A)to_float(y[n * ys]);
    if (bias) v += (A)to_float(bias[n]);
    y[n * ys] = Conv<T>::from(v);
  }
}
// The same product for rows that fit a wave's registers (K <= NL * 64 * V): a wave owns OPW outputs and issues every
// load of W and x before the first use, so one trip to memory covers the whole row; a decode step's projections
// against k-contiguous weights run at the cost of a streaming read.
// PRO_LN: the row multiplied is layer_norm(x; lnGain, lnBias) over its K elements -- every wave normalises the row it has
// loaded anyway (the routine the row kernel runs, so the same bits), and the first wave of the grid also stores it to lnOut,
// where the separate layer_norm op would have put it.
// PRO == 2: the row multiplied is the output of an attention whose key range was cut up -- every wave merges the parts'
// records into the piece of the row it needs (the routine the attention's own merge kernel runs, so the same bits), and the
// first wave of the grid also stores the row where that kernel would have put it (x is then only written, as am.out).
struct AttnMergeArgs { const float* partial = nullptr; int D = 0, logD = 0; void* out = nullptr; };
// STREAM: W comes through non-temporal loads -- the host asks for it when W is large against the last-level cache (a
// vocabulary's embedding under the logits of a decode step, 77 MB), so that one pass over it does not push out what the next
// step reads again (the layers' weights: batch-1 step 0.305 -> 0.279 ms)
template <typename T, int OPW, int NL, bool HAS_BIAS, int PRO = 0, bool STREAM = false>
__global__ __launch_bounds__(256) void gemv_rowdot_pre(const T* __restrict__ W, LongType ldw, const T* __restrict__ x, T* __restrict__ y, LongType ys,
                                                       LongType N, LongType K, const T* __restrict__ bias, int hasEpi, GemmEpilogue epi,
                                                       const T* __restrict__ lnGain = nullptr, const T* __restrict__ lnBias = nullptr,
                                                       T* __restrict__ lnOut = nullptr, float lnEps = 0.f, AttnMergeArgs am = AttnMergeArgs()) {
  constexpr bool PRO_LN = PRO == 1;
  constexpr int V = 16 / sizeof(T);
  using Raw = typename RawIO<T>::raw;
  const int lane = threadIdx.x & 63;
  const LongType n0 = ((LongType)blockIdx.x * 4 + (threadIdx.x >> 6)) * OPW;
  if (n0 >= N) return;
  const int kw = (int)(K / V);
  // Every load is unconditional -- lanes past the end of the row re-read its last word and their x bits are masked
  // to zero -- so that all of them are issued back to back rather than one predicated region (and one wait) per pass.
  raw_u32x4 wr[OPW][NL], xr[NL];
  const T* wrow[OPW];
#pragma unroll
  for (int o = 0; o < OPW; o++) wrow[o] = W + (n0 + o < N ? n0 + o : N - 1) * ldw;
#pragma unroll
  for (int i = 0; i < NL; i++) {
    const int kk = lane + 64 * i, kc = kk < kw ? kk : kw - 1;
#pragma unroll
    for (int o = 0; o < OPW; o++) {
      if constexpr (STREAM) wr[o][i] = __builtin_nontemporal_load(reinterpret_cast<const raw_u32x4*>(wrow[o]) + kc);
      else wr[o][i] = reinterpret_cast<const raw_u32x4*>(wrow[o])[kc];
    }
    if constexpr (PRO != 2) xr[i] = reinterpret_cast<const raw_u32x4*>(x)[kc];
  }
  if constexpr (PRO == 2) {
    const bool first = blockIdx.x == 0 && (threadIdx.x >> 6) == 0;
#pragma unroll
    for (int i = 0; i < NL; i++) {
      const int kk = lane + 64 * i, kc = kk < kw ? kk : kw - 1;
      // (four parts and a head size that is a power of two -- the host checks both -- keep this prologue one short code path)
      const int k = kc * V, head = k >> am.logD, t0 = k - (head << am.logD);
      float vals[V];
      attn_merge_parts<V, 4>(am.partial + (LongType)head * 4 * ATTN_PART_PITCH(am.D), am.D, t0, vals);
      const Raw packed = RawIO<T>::pack(vals);
      xr[i] = __builtin_bit_cast(raw_u32x4, packed);
      if (first && kk < kw) reinterpret_cast<Raw*>(am.out)[kk] = packed;
    }
  }
  T bq[OPW];
  if (HAS_BIAS) {
#pragma unroll
    for (int o = 0; o < OPW; o++) bq[o] = bias[n0 + o < N ? n0 + o : N - 1];
  }
  if (PRO_LN) {
    Raw gv[NL], bv[NL];
    float keepf[NL], vals[NL * V];
#pragma unroll
    for (int i = 0; i < NL; i++) {
      const int kk = lane + 64 * i, kc = kk < kw ? kk : kw - 1;
      gv[i] = reinterpret_cast<const Raw*>(lnGain)[kc];
      bv[i] = reinterpret_cast<const Raw*>(lnBias)[kc];
      keepf[i] = kk < kw ? 1.f : 0.f;
      RawIO<T>::unpack(__builtin_bit_cast(Raw, xr[i]), &vals[i * V]);
    }
    ln_wave_row<T, NL, true>(vals, gv, bv, keepf, (int)K, lnEps);
    const bool first = blockIdx.x == 0 && (threadIdx.x >> 6) == 0;
#pragma unroll
    for (int i = 0; i < NL; i++) {
      const Raw packed = RawIO<T>::pack(&vals[i * V]);
      xr[i] = __builtin_bit_cast(raw_u32x4, packed);
      if (first && lane + 64 * i < kw) reinterpret_cast<Raw*>(lnOut)[lane + 64 * i] = packed;
    }
  }
  // the bias enters lane 0's partial sum ahead of the wave reduction: a use every lane depends on, so its load stays
  // up here with the others instead of sinking into the one-lane store at the end
  float acc[OPW];
#pragma unroll
  for (int o = 0; o < OPW; o++) acc[o] = HAS_BIAS && lane == 0 ? to_float(bq[o]) : 0.f;
#pragma unroll
  for (int i = 0; i < NL; i++) {
    const unsigned keep = lane + 64 * i < kw ? 0xffffffffu : 0u;
    const raw_u32x4 xm = xr[i] & keep;
    float xf[V];
    RawIO<T>::unpack(__builtin_bit_cast(Raw, xm), xf);
#pragma unroll
    for (int o = 0; o < OPW; o++) {
      float wf[V];
      RawIO<T>::unpack(__builtin_bit_cast(Raw, wr[o][i]), wf);
#pragma unroll
      for (int e = 0; e < V; e++) acc[o] = fmaf(wf[e], xf[e], acc[o]);
    }
  }
#pragma unroll
  for (int o = 0; o < OPW; o++) {
    const float v = wave_allreduce<SumOp>(acc[o]);
    if (lane == 0 && n0 + o < N) {
      const T yv = Conv<T>::from(v);
      y[(n0 + o) * ys] = yv;
      epilogueExtras<T>(hasEpi, epi, 0, n0 + o, yv);
    }
  }
}
template <typename T>
static bool tryGemvRowdotPre(hipStream_t s, const GemmDesc& d, const void* A, const void* B, void* C) {
  constexpr int V = 16 / sizeof(T);
  if (d.aCol != 1 || d.alpha != 1.f || d.beta != 0.f || d.K % V != 0 || d.bCol % V != 0) return false;
  if ((reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(B)) & 15) return false;
  const LongType passes = (d.K / V + 63) / 64;
  const bool stream = (double)d.N * (double)d.K * sizeof(T) >= (double)(32 << 20);
#define ROWDOT_BS(OPW, NL, HB, ST) hipLaunchKernelGGL((gemv_rowdot_pre<T, OPW, NL, HB, 0, ST>), dim3((unsigned)(((d.N + OPW - 1) / OPW + 3) / 4)), dim3(256), 0, s, \
                                                      (const T*)B, d.bCol, (const T*)A, (T*)C, d.cCol, d.N, d.K, (const T*)d.bias, d.epi ? 1 : 0, d.epi ? *d.epi : GemmEpilogue())
#define ROWDOT_B(OPW, NL, HB) do { if (stream) ROWDOT_BS(OPW, NL, HB, true); else ROWDOT_BS(OPW, NL, HB, false); } while (0)
#define ROWDOT_LN(OPW, NL) hipLaunchKernelGGL((gemv_rowdot_pre<T, OPW, NL, true, true>), dim3((unsigned)(((d.N + OPW - 1) / OPW + 3) / 4)), dim3(256), 0, s, \
                                              (const T*)B, d.bCol, (const T*)A, (T*)C, d.cCol, d.N, d.K, (const T*)d.bias, d.epi ? 1 : 0, d.epi ? *d.epi : GemmEpilogue(), \
                                              (const T*)d.lnGain, (const T*)d.lnBias, (T*)d.lnOut, d.lnEps)
#define ROWDOT_AM(OPW, NL) hipLaunchKernelGGL((gemv_rowdot_pre<T, OPW, NL, true, 2>), dim3((unsigned)(((d.N + OPW - 1) / OPW + 3) / 4)), dim3(256), 0, s, \
                                              (const T*)B, d.bCol, (const T*)A, (T*)C, d.cCol, d.N, d.K, (const T*)d.bias, d.epi ? 1 : 0, d.epi ? *d.epi : GemmEpilogue(), \
                                              (const T*)nullptr, (const T*)nullptr, (T*)nullptr, 0.f, am)
#define ROWDOT(OPW, NL) do { noteKernel("gemv_rowdot_pre<%s,opw=%d,nl=%d>", tname<T>(), OPW, NL); if (d.bias) ROWDOT_B(OPW, NL, true); else ROWDOT_B(OPW, NL, false); } while (0)
  if (d.attnPartial) {   // the row is merged from the records of a cut-up attention on the way in: short rows with a bias only
    if (!d.bias || passes > 2 || d.attnSplits != 4 || (d.attnD != 64 && d.attnD != 128) || d.K % d.attnD != 0 || (reinterpret_cast<uintptr_t>(d.attnOut) & 15)) return false;
    AttnMergeArgs am;
    am.partial = d.attnPartial; am.D = d.attnD; am.logD = d.attnD == 64 ? 6 : 7; am.out = d.attnOut;
    noteKernel("gemv_rowdot_pre<%s,attn-merge,nl=2>", tname<T>());
    ROWDOT_AM(2, 2);
    return true;
  }
  if (d.lnGain) {   // the row is normalised on the way in: short rows with a bias only
    if (!d.bias || passes > 4 || ((reinterpret_cast<uintptr_t>(d.lnGain) | reinterpret_cast<uintptr_t>(d.lnBias) | reinterpret_cast<uintptr_t>(d.lnOut)) & 15)) return false;
    noteKernel("gemv_rowdot_pre<%s,ln,nl=%d>", tname<T>(), passes <= 2 ? 2 : 4);
    if (passes <= 2) ROWDOT_LN(2, 2); else ROWDOT_LN(2, 4);
    return true;
  }
  if (passes <= 2) ROWDOT(2, 2);
  else if (passes <= 4) ROWDOT(2, 4);
  else if (passes <= 6) ROWDOT(2, 6);
  else if (passes <= 8) ROWDOT(2, 8);
  else if (passes <= 12) ROWDOT(1, 12);
  else return false;
#undef ROWDOT
#undef ROWDOT_B
#undef ROWDOT_BS
#undef ROWDOT_LN
#undef ROWDOT_AM
  return true;
}
// y[n] = alpha * sum_k x[k] * W[k][n]: W rows contiguous in n.  A thread owns V consecutive outputs of one k-slice;
// slices are combined through LDS (block = 64 column groups x 4 k-slices).
template <typename T>
__global__ __launch_bounds__(256) void gemv_colsum(const T* __restrict__ W, LongType ldw, const T* __restrict__ x, LongType xs, T* __restrict__ y,
                                                   LongType ys, LongType N, LongType K, float alpha, float beta, const T* __restrict__ bias) {
  using A = typename Conv<T>::acc;
  constexpr int V = 16 / sizeof(T);
  using VT = Vec<T, V>;
  __shared__ A part[4][64 * V];
  const int cg = threadIdx.x & 63, slice = threadIdx.x >> 6;
  const LongType n0 = ((LongType)blockIdx.x * 64 + cg) * V;
  A acc[V];
#pragma unroll
  for (int e = 0; e < V; e++) acc[e] = 0;
  if (n0 < N) {
    const bool vec = N % V == 0 && ldw % V == 0 && (reinterpret_cast<uintptr_t>(W) & 15) == 0;
    for (LongType k = slice; k < K; k += 4) {
      const A xv = (A)to_float(x[k * xs]);
      if (vec) {
        VT w = *reinterpret_cast<const VT*>(W + k * ldw + n0);
#pragma unroll
        for (int e = 0; e < V; e++) acc[e] += xv * (A)to_float(w.v[e]);
      } else {
#pragma unroll
        for (int e = 0; e < V; e++) if (n0 + e < N) acc[e] += xv * (A)to_float(W[k * ldw + n0 + e]);
      }
    }
  }
#pragma unroll
  for (int e = 0; e < V; e++) part[slice][cg * V + e] = acc[e];
  __syncthreads();
  if (slice == 0 && n0 < N) {
#pragma unroll
    for (int e = 0; e < V; e++) {
      if (n0 + e >= N) break;
      A v = (A)alpha * (part[0][cg * V + e] + part[1][cg * V + e] + part[2][cg * V + e] + part[3][cg * V + e]);
      if (beta != 0.f) v += (A)beta * (A)to_float(y[(n0 + e) * ys]);
      if (bias) v += (A)to_float(bias[n0 + e]);
      y[(n0 + e) * ys] = Conv<T>::from(v);
    }
  }
}

template <typename T>
static bool tryGemv(hipStream_t s, const GemmDesc& d, const void* A, const void* B, void* C) {
  if (d.batch != 1) return false;
  constexpr int V = 16 / sizeof(T);
  if (d.M == 1 && d.N > 1) {
    // y[n] = sum_k a[k] * op(B)[k][n]
    if (d.bRow == 1 && (!d.epi || d.cCol == 1) && tryGemvRowdotPre<T>(s, d, A, B, C)) return true;
    if (d.epi) return false;
    if (d.bRow == 1) { noteKernel("gemv_rowdot<%s>", tname<T>()); hipLaunchKernelGGL((gemv_rowdot<T>), dim3((unsigned)((d.N + 3) / 4)), dim3(256), 0, s, (const T*)B, d.bCol, (const T*)A, d.aCol, (T*)C, d.cCol, d.N, d.K, d.alpha, d.beta, (const T*)d.bias); return true; }
    if (d.bCol == 1) { noteKernel("gemv_colsum<%s>", tname<T>()); hipLaunchKernelGGL((gemv_colsum<T>), dim3((unsigned)((d.N + 64 * V - 1) / (64 * V))), dim3(256), 0, s, (const T*)B, d.bRow, (const T*)A, d.aCol, (T*)C, d.cCol, d.N, d.K, d.alpha, d.beta, (const T*)d.bias); return true; }
  }
  if (d.N == 1 && d.M > 1 && !d.bias && !d.epi) {
    // y[m] = sum_k op(A)[m][k] * b[k]
    if (d.aCol == 1) { noteKernel("gemv_rowdot<%s>", tname<T>()); hipLaunchKernelGGL((gemv_rowdot<T>), dim3((unsigned)((d.M + 3) / 4)), dim3(256), 0, s, (const T*)A, d.aRow, (const T*)B, d.bRow, (T*)C, d.cRow, d.M, d.K, d.alpha, d.beta, (const T*)nullptr); return true; }
    if (d.aRow == 1) { noteKernel("gemv_colsum<%s>", tname<T>()); hipLaunchKernelGGL((gemv_colsum<T>), dim3((unsigned)((d.M + 64 * V - 1) / (64 * V))), dim3(256), 0, s, (const T*)A, d.aCol, (const T*)B, d.bRow, (T*)C, d.cRow, d.M, d.K, d.alpha, d.beta, (const T*)nullptr); return true; }
  }
  return false;
}

// ---- dispatch ---------------------------------------------------------------------------------------------------------
static GemmArgs toArgs(const GemmDesc& d) {
  GemmArgs g;
  g.M = d.M; g.N = d.N; g.K = d.K;
  g.aRow = d.aRow; g.aCol = d.aCol; g.bRow = d.bRow; g.bCol = d.bCol; g.cRow = d.cRow; g.cCol = d.cCol;
  g.aBatch = d.aBatch; g.bBatch = d.bBatch; g.cBatch = d.cBatch;
  g.batchInner = d.batchInner; g.aBatch2 = d.aBatch2; g.bBatch2 = d.bBatch2; g.cBatch2 = d.cBatch2;
  g.alpha = d.alpha; g.beta = d.beta;
  g.splits = 1; g.ktPerSplit = 0; g.partial = nullptr; g.bias = d.bias;
  g.hasEpi = d.epi ? 1 : 0;
  if (d.epi) g.epi = *d.epi;
  g.lnGain = d.lnGain; g.lnBias = d.lnBias; g.lnOut = d.lnOut; g.lnOutRow = d.lnOutRow; g.lnEps = d.lnEps;
  return g;
}

template <typename T>
static void launchSimple(hipStream_t s, const void* A, const void* B, void* C, const GemmDesc& d) {
  GemmArgs g = toArgs(d);
  dim3 grid((unsigned)((d.N + 31) / 32), (unsigned)((d.M + 31) / 32), (unsigned)d.batch);
  noteKernel("gemm_simple<%s>", tname<T>());
  hipLaunchKernelGGL((gemm_simple<T>), grid, dim3(256), 0, s, g, (const T*)A, (const T*)B, (T*)C);
}

// can the MFMA kernels take this problem: 16-byte aligned vectors along each operand's contiguous axis
// `aligned`: every operand vector the loaders fetch starts on a 16-byte boundary and the contiguous extents are whole vectors --
// what the direct-to-LDS kernels and the kernels without bounds handling need.  Without it only the kernels whose loader
// takes element-aligned rows and ragged extents (gemm_mfma16p, gemm_mfma16, gemm_mfma32) may run.
static bool mfmaEligible(const GemmDesc& d, const void* A, const void* B, size_t es, bool& aKC, bool& bKC, bool& aligned) {
  const LongType V = 16 / (LongType)es;
  if (d.M < 1 || d.N < 1 || d.K < V) return false;
  if (d.aRow < 0 || d.aCol < 0 || d.bRow < 0 || d.bCol < 0) return false;
  if (d.aCol == 1) aKC = true;
  else if (d.aRow == 1 && d.M >= V) aKC = false;
  else return false;
  if (d.bRow == 1) bKC = true;
  else if (d.bCol == 1 && d.N >= V) bKC = false;
  else return false;
  aligned = ((reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(B)) & 15) == 0;
  if (d.batch > 1 && (d.aBatch % V || d.bBatch % V)) aligned = false;
  if (d.batchInner > 0 && (d.aBatch2 % V || d.bBatch2 % V)) aligned = false;
  if (aKC ? (d.K % V != 0 || d.aRow % V != 0) : (d.M % V != 0 || d.aCol % V != 0)) aligned = false;
  if (bKC ? (d.K % V != 0 || d.bCol % V != 0) : (d.N % V != 0 || d.bRow % V != 0)) aligned = false;
  return true;
}

// ---- up to four rows of x against row-major W (a decode step's projections) --------------------------------------------------
// One block per strip of CW output columns and all of K: a lane loads 8 neighbouring columns of one k-row (16 bytes), a wave
// covers 64/(CW/8) k-rows per instruction, the waves interleave rows, and a lane issues up to eight independent loads before
// it touches the first.  Narrow strips (CW = 8: N/8 blocks) spread the weights over every CU -- one CU streams only at its
// share of the bandwidth -- and the XCD-aware strip order lets the blocks that share a weight row's cache lines hit the same
// L2.  x sits in LDS.  Partial sums meet through lane shuffles (rows of a wave) and LDS (waves), in a fixed order.  One
// launch, no partial tiles in global memory.
template <typename T, int M, int CW, int NWAVE>
__global__ __launch_bounds__(NWAVE * 64) void gemv_strip(GemmArgs g, const T* __restrict__ x, const T* __restrict__ W, T* __restrict__ out) {
  constexpr int LPR = CW / 8, RPW = 64 / LPR, RB = NWAVE * RPW;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  float* red = reinterpret_cast<float*>(smem_raw);                      // [16 waves][M][CW]
  T* xs = reinterpret_cast<T*>(red + NWAVE * M * CW);                    // [M][K]
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6, cg = lane % LPR, rk = lane / LPR;
  const LongType K = g.K;
  // consecutive block ids sit on different XCDs: give every XCD a run of neighbouring strips, so that strips which share
  // 128-byte lines of a weight row are served by one L2
  unsigned strip;
  {
    const unsigned total = gridDim.x, xcd = blockIdx.x & 7u, idx = blockIdx.x >> 3, per = total >> 3, rem = total & 7u;
    strip = xcd * per + (xcd < rem ? xcd : rem) + idx;
  }
  const LongType c0 = (LongType)strip * CW + cg * 8;
  const T* wp = W + (LongType)(wave * RPW + rk) * g.bRow + c0;
  const LongType step = (LongType)RB * g.bRow;
  LongType k = wave * RPW + rk;
  // the first batch of weight loads goes out before x is staged
  u32x4 w[8];
  const int first = (int)((K - k + RB - 1) / RB < 8 ? (K - k + RB - 1) / RB : 8);
#pragma unroll
  for (int i = 0; i < 8; i++)
    if (i < first) w[i] = *reinterpret_cast<const u32x4*>(wp + i * step);
  for (LongType i = t; i < (LongType)M * K; i += NWAVE * 64) {
    const LongType m = i / K, kk = i - m * K;
    xs[i] = x[m * g.aRow + kk];
  }
  __syncthreads();
  float acc[M][8];
#pragma unroll
  for (int m = 0; m < M; m++)
#pragma unroll
    for (int e = 0; e < 8; e++) acc[m][e] = 0.f;
  auto fma8 = [&](const u32x4& wq, LongType kk) {
    float wv[8];
#pragma unroll
    for (int q = 0; q < 4; q++) {
      wv[2 * q] = to_float(__builtin_bit_cast(T, (unsigned short)(wq[q] & 0xffffu)));
      wv[2 * q + 1] = to_float(__builtin_bit_cast(T, (unsigned short)(wq[q] >> 16)));
    }
#pragma unroll
    for (int m = 0; m < M; m++) {
      const float xv = to_float(xs[(LongType)m * K + kk]);
#pragma unroll
      for (int e = 0; e < 8; e++) acc[m][e] = fmaf(xv, wv[e], acc[m][e]);
    }
  };
  int have = first;
  while (have > 0) {
    const LongType kNext = k + (LongType)have * RB;
    const T* wpNext = wp + (LongType)have * step;
    u32x4 nw[8];
    const int more = (int)((K - kNext + RB - 1) / RB < 8 ? (kNext < K ? (K - kNext + RB - 1) / RB : 0) : 8);
#pragma unroll
    for (int i = 0; i < 8; i++)
      if (i < more) nw[i] = *reinterpret_cast<const u32x4*>(wpNext + i * step);
#pragma unroll
    for (int i = 0; i < 8; i++)
      if (i < have) fma8(w[i], k + (LongType)i * RB);
#pragma unroll
    for (int i = 0; i < 8; i++) w[i] = nw[i];
    k = kNext; wp = wpNext; have = more;
  }
  // rows of the wave: lanes that share a column group
#pragma unroll
  for (int off = LPR; off < 64; off <<= 1)
#pragma unroll
    for (int m = 0; m < M; m++)
#pragma unroll
      for (int e = 0; e < 8; e++) acc[m][e] += __shfl_xor(acc[m][e], off, 64);
  if (rk == 0) {
#pragma unroll
    for (int m = 0; m < M; m++)
#pragma unroll
      for (int e = 0; e < 8; e++) red[(wave * M + m) * CW + cg * 8 + e] = acc[m][e];
  }
  __syncthreads();
  if (t < M * CW) {
    const int m = t / CW, c = t % CW;
    float v = 0.f;
#pragma unroll
    for (int q = 0; q < NWAVE; q++) v += red[(q * M + m) * CW + c];
    const LongType col = (LongType)strip * CW + c;
    if (g.bias) v += to_float(static_cast<const T*>(g.bias)[col]);
    out[(LongType)m * g.cRow + col] = Conv<T>::from(v);
  }
}
template <typename T, int M>
static void launchGemvStripM(hipStream_t s, const GemmArgs& g, const void* A, const void* B, void* C) {
  // strips of 8 columns (one 16-byte piece of every weight row): N/8 blocks keep every CU busy even for N = 768
  constexpr int CW = 8, NWAVE = 4;
  const size_t lds = (size_t)NWAVE * M * CW * sizeof(float) + (size_t)M * g.K * sizeof(T);
  noteKernel("gemv_strip<%s,m=%d>", tname<T>(), M);
  hipLaunchKernelGGL((gemv_strip<T, M, CW, NWAVE>), dim3((unsigned)(g.N / CW)), dim3(NWAVE * 64), lds, s, g, (const T*)A, (const T*)B, (T*)C);
}
// whether the strip kernel takes this product: a few dense rows, W row-major with aligned rows, plain C = A B (+ bias)
template <typename T>
static bool tryGemvStrip(hipStream_t s, const GemmDesc& d, const void* A, const void* B, void* C) {
  if (d.M < 1 || d.M > 4 || d.batch != 1 || d.alpha != 1.f || d.beta != 0.f || d.epi) return false;
  if (d.aCol != 1 || d.bCol != 1 || d.cCol != 1 || d.bRow % 8 != 0) return false;
  if (d.N % 32 != 0 || d.K % 256 != 0 || d.N < 256) return false;
  if ((reinterpret_cast<uintptr_t>(B) & 15) != 0) return false;
  if ((size_t)4 * d.M * 8 * sizeof(float) + (size_t)d.M * d.K * sizeof(T) > 60 * 1024) return false;
  GemmArgs g = toArgs(d);
  switch (d.M) {
    case 1: launchGemvStripM<T, 1>(s, g, A, B, C); break;
    case 2: launchGemvStripM<T, 2>(s, g, A, B, C); break;
    case 3: launchGemvStripM<T, 3>(s, g, A, B, C); break;
    default: launchGemvStripM<T, 4>(s, g, A, B, C); break;
  }
  return true;
}

// ---- up to 32 rows of x against k-contiguous weights (a batched decode step's projections) -----------------------------
// C[m][n] = sum_k x[m][k] * Wt[n][k] (+ bias[n]).  A block owns 32 output columns and all of K, in chunks of up to 384 k
// (two chunks for d_model = 768; the LDS footprint stays under 64 KiB, which every launch path -- graph kernel nodes
// included -- takes without a raised per-function limit):
// every thread issues the chunk's loads at once (whole 128-byte lines: 8 lanes per row), parks them in LDS in the
// [k-group][row] slot layout, and the four waves share the chunk's MFMA k-steps; the next chunk's loads are in flight
// while the current one is multiplied.  The waves' 32x32 partial tiles are added up through LDS -- one launch, where the
// split-K tile kernel needs a second one to add its partial tiles.
// Accumulator layout: lane (m = lane % 32, h = lane / 32), register r holds column 8 * (r / 4) + 4 * h + r % 4.
// LN_NV > 0: the rows of X are layer-normalised over K on the way in (and block 0 writes the normalised rows to g.lnOut),
// with the bits of the separate layer_norm kernel, which gives a wave to a row: lane l of that wave sums the 8-value
// vectors l and l + 64 of the row (LN_NV = 2 passes; one pass for K <= 512), then the wave adds its lanes up as a balanced
// tree over the lane numbers.  Here the 8 threads of a row hold vector 8 * tile + lkg of every tile, so thread lkg stands in
// for that wave's lanes 8 * jj + lkg, jj = 0..7: the first three levels of the tree run across the 8 threads (the same lane
// exchanges), the last three inside a thread over jj.  Everything else of the normalisation is per element.  Needs the
// whole row in registers: K <= 768.
template <typename T, int LN_NV = 0>
__global__ __launch_bounds__(256) void gemm_skinny32(GemmArgs g, const T* __restrict__ X, const T* __restrict__ Wt, T* __restrict__ C) {
  constexpr int CT = 6;                                // 64-k tiles per chunk
  constexpr int GROUP = 33;                            // slots per k-group (32 rows + 1: conflict-free column reads)
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  u32x4* sW = reinterpret_cast<u32x4*>(smem_raw);      // [CT * 8 k-groups][GROUP]
  u32x4* sX = sW + CT * 8 * GROUP;
  float* red = reinterpret_cast<float*>(smem_raw);     // [4 waves][16 registers][64 lanes]; reuses sW once the K loop is over
  const int t = threadIdx.x, lane = t & 63, wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const int lrow = t >> 3, lkg = t & 7;                // this thread's (row, k-group) inside every 64-k tile
  const LongType n0 = (LongType)blockIdx.x * 32;
  const T* wp = Wt + (n0 + lrow) * g.bCol + lkg * 8;
  const T* xp = X + (LongType)(lrow < g.M ? lrow : g.M - 1) * g.aRow + lkg * 8;
  const int tiles = (int)(g.K / 64);
  // two register sets: the loads of two chunks are on their way at any time, so that K = 768 (two chunks) costs one trip
  // to memory, not two -- the second chunk's latency was a quarter of the kernel's time
  u32x4 wr[2][CT], xr[2][CT];
  auto load = [&](int set, int tile0) {
    const int n = tiles - tile0 < CT ? tiles - tile0 : CT;
#pragma unroll
    for (int j = 0; j < CT; j++) {
      const int jc = j < n ? j : n - 1;                // unconditional loads; a repeated tile is never multiplied
      wr[set][j] = *reinterpret_cast<const u32x4*>(wp + (LongType)(tile0 + jc) * 64);
      xr[set][j] = *reinterpret_cast<const u32x4*>(xp + (LongType)(tile0 + jc) * 64);
    }
  };
  f32x16 acc;
#pragma unroll
  for (int r = 0; r < 16; r++) acc[r] = 0.f;
  const int mrow = lane & 31, h = lane >> 5;
  if constexpr (LN_NV == 0) {
    load(0, 0);
    if (CT < tiles) load(1, CT);
  }
  if constexpr (LN_NV > 0) {
    using IO = RawIO<T>;
    using Raw = typename IO::raw;
    // gain and bias go through LDS (a stage of their own behind the chunk stages): 2 x K / 8 vector loads per block instead
    // of 24 per thread, and no registers held for them while the row is normalised
    u32x4* sGB = sW + 2 * CT * 8 * GROUP;                  // [2][128] vectors: gain, then bias
    // loads come back in the order they were issued: the rows (written by the kernel before this one, so close by), gain
    // and bias go first and the weights, which come from far away, last -- the normalisation then runs while they travel
#pragma unroll
    for (int j = 0; j < 2 * CT; j++) {
      const int jc = j < tiles ? j : tiles - 1;
      xr[j / CT][j % CT] = *reinterpret_cast<const u32x4*>(xp + (LongType)jc * 64);
    }
    {
      const int v = t & 127, vc = v < tiles * 8 ? v : tiles * 8 - 1;
      const T* src = reinterpret_cast<const T*>(t < 128 ? g.lnGain : g.lnBias) + vc * 8;
      sGB[t] = *reinterpret_cast<const u32x4*>(src);
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int j = 0; j < 2 * CT; j++) {
      const int jc = j < tiles ? j : tiles - 1;
      wr[j / CT][j % CT] = *reinterpret_cast<const u32x4*>(wp + (LongType)jc * 64);
    }
    __builtin_amdgcn_sched_barrier(0);
    // the row's total of f(vector), f evaluated per tile into part[]: per stand-in lane the passes in order (a lane past
    // the row's end adds the row's last vector times zero, as the separate kernel's lanes do), then the tree
    auto rowTotal = [&](const float (&part)[2 * CT]) {
      float last = 0.f;
#pragma unroll
      for (int j = 0; j < 2 * CT; j++) if (j == tiles - 1) last = part[j];
      last = __shfl(last, lane | 7, 64);                  // the row's last vector sits with lkg = 7
      float o[8];
#pragma unroll
      for (int jj = 0; jj < 8; jj++) {
        float s = 0.f;
#pragma unroll
        for (int i = 0; i < LN_NV; i++) {
          const int tile = jj + 8 * i;
          const bool in = tile < tiles;
          const float p = tile < 2 * CT && in ? part[tile < 2 * CT ? tile : 0] : last;
          s += p * (in ? 1.f : 0.f);
        }
        o[jj] = group_allreduce<SumOp, 8>(s);
      }
      return ((o[0] + o[1]) + (o[2] + o[3])) + ((o[4] + o[5]) + (o[6] + o[7]));
    };
    // the row in fp32, kept in registers through the three passes
    float part[2 * CT], vals[2 * CT][8];
#pragma unroll
    for (int j = 0; j < 2 * CT; j++) {
      IO::unpack(__builtin_bit_cast(Raw, xr[j / CT][j % CT]), vals[j]);
      float p = 0.f;
#pragma unroll
      for (int e = 0; e < 8; e++) p += vals[j][e];
      part[j] = p;
    }
    const float mean = rowTotal(part) / (float)(int)g.K;
#pragma unroll
    for (int j = 0; j < 2 * CT; j++) {
      float p = 0.f;
#pragma unroll
      for (int e = 0; e < 8; e++) { const float d = vals[j][e] - mean; vals[j][e] = d; p += d * d; }
      part[j] = p;
    }
    const float var = rowTotal(part) / (float)(int)g.K;
    const float rstd = 1.f / sqrtf(var + g.lnEps);
    const bool writer = blockIdx.x == 0 && lrow < g.M;
    T* lo = reinterpret_cast<T*>(g.lnOut) + (LongType)lrow * g.lnOutRow + lkg * 8;
    __syncthreads();                                       // gain and bias are in LDS
#pragma unroll
    for (int j = 0; j < 2 * CT; j++) {
      float gn[8], bs[8];
      const int vj = j < tiles ? j * 8 + lkg : 0;
      IO::unpack(__builtin_bit_cast(Raw, sGB[vj]), gn);
      IO::unpack(__builtin_bit_cast(Raw, sGB[128 + vj]), bs);
#pragma unroll
      for (int e = 0; e < 8; e++) {
        float y = vals[j][e] * rstd * gn[e];
        y += bs[e];
        vals[j][e] = y;
      }
      const Raw packed = IO::pack(vals[j]);
      xr[j / CT][j % CT] = __builtin_bit_cast(u32x4, packed);
      if (writer && j < tiles) *reinterpret_cast<Raw*>(lo + j * 64) = packed;
    }
  }
  auto chunk = [&](int set, int tile0) {
    const int n = tiles - tile0 < CT ? tiles - tile0 : CT;
#pragma unroll
    for (int j = 0; j < CT; j++) {
      sW[(j * 8 + lkg) * GROUP + lrow] = wr[set][j];
      sX[(j * 8 + lkg) * GROUP + lrow] = xr[set][j];
    }
    __syncthreads();
    if (tile0 + 2 * CT < tiles) load(set, tile0 + 2 * CT);
    for (int s = wave; s < n * 4; s += 4)
      acc = Mfma16<T>::mma(sW[(2 * s + h) * GROUP + mrow], sX[(2 * s + h) * GROUP + mrow], acc);
    __syncthreads();
  };
  for (int tile0 = 0; tile0 < tiles; tile0 += 2 * CT) {
    chunk(0, tile0);
    if (tile0 + CT < tiles) chunk(1, tile0 + CT);
  }
#pragma unroll
  for (int r = 0; r < 16; r++) red[(wave * 16 + r) * 64 + lane] = acc[r];
  __syncthreads();
  const int rq = wave;                                 // registers 4 * rq .. + 3: four consecutive columns
  const LongType n = n0 + 8 * rq + 4 * h;
  float v[4];
#pragma unroll
  for (int e = 0; e < 4; e++) {
    float sum = 0.f;
#pragma unroll
    for (int w = 0; w < 4; w++) sum += red[(w * 16 + 4 * rq + e) * 64 + lane];
    if (g.bias) sum += to_float(reinterpret_cast<const T*>(g.bias)[n + e]);
    v[e] = sum;
  }
  if (mrow < g.M) {
    u32x2 o;
    o[0] = (unsigned)Conv<T>::from(v[0]).bits | ((unsigned)Conv<T>::from(v[1]).bits << 16);
    o[1] = (unsigned)Conv<T>::from(v[2]).bits | ((unsigned)Conv<T>::from(v[3]).bits << 16);
    *reinterpret_cast<u32x2*>(C + (LongType)mrow * g.cRow + n) = o;
    epilogueExtras4<T>(g, mrow, n, v);
  }
}
// The layer-normalising few-row product with the rows cut in two: a block owns 32 output columns and 16 rows (grid: N / 32 x
// ceil(M / 16)).  Every block of gemm_skinny32 normalises all 32 rows before it can multiply -- 96 values per thread, vector
// ALU work at one wave per SIMD, 3.4 us of the kernel's 8.4 and the same in every block.  With 16 rows a thread holds 48
// values, and twice as many CUs share the step's work; the weights are read by two blocks instead of one (from the cache).
// 16 threads hold a row: thread lk16 of them holds vector 16 * t2 + lk16, t2 = 0..5, and stands in for lane
// 16 * (t2 % 4) + lk16 of the separate layer_norm kernel's wave in its pass t2 / 4 -- the first four levels of that wave's
// balanced tree run across the 16 threads, the last two inside a thread, so the statistics carry the same bits.
// Rows 16..31 of the matrix instruction's X operand are whatever LDS holds: a row of the product depends on its own row of
// X only, and those rows are not stored.
template <typename T, int LN_NV, int ROWS = 16>
__global__ __launch_bounds__(256) void gemm_skinny16ln(GemmArgs g, const T* __restrict__ X, const T* __restrict__ Wt, T* __restrict__ C) {
  static_assert(ROWS == 16 || ROWS == 8, "rows per block");
  constexpr int CT = 6, GROUP = 33;
  constexpr int TPR = 256 / ROWS, XV = 96 / TPR, JJ = 64 / TPR;   // threads per row, vectors per thread, stand-in lanes per thread
  using IO = RawIO<T>;
  using Raw = typename IO::raw;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  u32x4* sW = reinterpret_cast<u32x4*>(smem_raw);      // [CT * 8 k-groups][GROUP]
  u32x4* sX = sW + CT * 8 * GROUP;
  u32x4* sGB = sW + 2 * CT * 8 * GROUP;                // [2][128] vectors: gain, then bias
  float* red = reinterpret_cast<float*>(smem_raw);     // [4 waves][16 registers][64 lanes]; reuses sW once the K loop is over
  const int t = threadIdx.x, lane = t & 63, wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const int lrow = t >> 3, lkg = t & 7;                // W: this thread's (column, k-group) inside every 64-k tile
  const int xr16 = t / TPR, lk16 = t % TPR;            // X: this thread's row of the block's ROWS and its vector index mod TPR
  const LongType n0 = (LongType)blockIdx.x * 32, m0 = (LongType)blockIdx.y * ROWS;
  const T* wp = Wt + (n0 + lrow) * g.bCol + lkg * 8;
  const T* xp = X + (m0 + xr16 < g.M ? m0 + xr16 : g.M - 1) * g.aRow;
  const int tiles = (int)(g.K / 64), nv = tiles * 8;
  u32x4 wr[2][CT], xv[XV];
#pragma unroll
  for (int t2 = 0; t2 < XV; t2++) {
    const int v = TPR * t2 + lk16;
    xv[t2] = *reinterpret_cast<const u32x4*>(xp + (LongType)(v < nv ? v : nv - 1) * 8);
  }
  {
    const int v = t & 127, vc = v < nv ? v : nv - 1;
    const T* src = reinterpret_cast<const T*>(t < 128 ? g.lnGain : g.lnBias) + vc * 8;
    sGB[t] = *reinterpret_cast<const u32x4*>(src);
  }
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int j = 0; j < 2 * CT; j++) {
    const int jc = j < tiles ? j : tiles - 1;
    wr[j / CT][j % CT] = *reinterpret_cast<const u32x4*>(wp + (LongType)jc * 64);
  }
  __builtin_amdgcn_sched_barrier(0);
  const int lastV = nv - 1, lastT2 = lastV / TPR, lastLk = lastV % TPR;
  auto rowTotal = [&](const float (&part)[XV]) {
    float last = 0.f;
#pragma unroll
    for (int t2 = 0; t2 < XV; t2++) if (t2 == lastT2) last = part[t2];
    last = __shfl(last, (lane & ~(TPR - 1)) | lastLk, 64);
    float o[JJ];
#pragma unroll
    for (int jj = 0; jj < JJ; jj++) {
      float s = 0.f;
#pragma unroll
      for (int i = 0; i < LN_NV; i++) {
        const int t2 = jj + JJ * i;
        const bool in = TPR * t2 + lk16 < nv;
        const float p = t2 < XV && in ? part[t2 < XV ? t2 : 0] : last;
        s += p * (in ? 1.f : 0.f);
      }
      o[jj] = group_allreduce<SumOp, TPR>(s);
    }
    if constexpr (JJ == 4) return (o[0] + o[1]) + (o[2] + o[3]);
    else return o[0] + o[1];
  };
  float part[XV], vals[XV][8];
#pragma unroll
  for (int t2 = 0; t2 < XV; t2++) {
    IO::unpack(__builtin_bit_cast(Raw, xv[t2]), vals[t2]);
    float p = 0.f;
#pragma unroll
    for (int e = 0; e < 8; e++) p += vals[t2][e];
    part[t2] = p;
  }
  const float mean = rowTotal(part) / (float)(int)g.K;
#pragma unroll
  for (int t2 = 0; t2 < XV; t2++) {
    float p = 0.f;
#pragma unroll
    for (int e = 0; e < 8; e++) { const float d = vals[t2][e] - mean; vals[t2][e] = d; p += d * d; }
    part[t2] = p;
  }
  const float var = rowTotal(part) / (float)(int)g.K;
  const float rstd = 1.f / sqrtf(var + g.lnEps);
  const bool writer = blockIdx.x == 0 && m0 + xr16 < g.M;
  T* lo = reinterpret_cast<T*>(g.lnOut) + (m0 + xr16) * g.lnOutRow;
  __syncthreads();                                       // gain and bias are in LDS
#pragma unroll
  for (int t2 = 0; t2 < XV; t2++) {
    float gn[8], bs[8];
    const int v = TPR * t2 + lk16, vj = v < nv ? v : 0;
    IO::unpack(__builtin_bit_cast(Raw, sGB[vj]), gn);
    IO::unpack(__builtin_bit_cast(Raw, sGB[128 + vj]), bs);
#pragma unroll
    for (int e = 0; e < 8; e++) {
      float y = vals[t2][e] * rstd * gn[e];
      y += bs[e];
      vals[t2][e] = y;
    }
    const Raw packed = IO::pack(vals[t2]);
    xv[t2] = __builtin_bit_cast(u32x4, packed);
    if (writer && v < nv) *reinterpret_cast<Raw*>(lo + (LongType)v * 8) = packed;
  }
  f32x16 acc;
#pragma unroll
  for (int r = 0; r < 16; r++) acc[r] = 0.f;
  const int mrow = lane & 31, h = lane >> 5;
  // chunk `set`: K-tiles set * CT .. + CT - 1 -- the W registers of that set and this thread's X vectors 3 * set .. + 2
  // (vector 16 * t2 + lk16 is k-group lk16 % 8 of K-tile 2 * t2 + lk16 / 8)
  auto chunk = [&](auto setc) {
    constexpr int set = decltype(setc)::value;
    const int n = tiles - set * CT < CT ? tiles - set * CT : CT;
#pragma unroll
    for (int j = 0; j < CT; j++) sW[(j * 8 + lkg) * GROUP + lrow] = wr[set][j];
#pragma unroll
    for (int t2 = 0; t2 < XV; t2++) {
      const int tile = (TPR * t2 + lk16) >> 3;   // the K-tile of this vector; k-group lk16 % 8
      if (tile / CT == set) sX[((tile - set * CT) * 8 + (lk16 & 7)) * GROUP + xr16] = xv[t2];
    }
    __syncthreads();
    for (int s = wave; s < n * 4; s += 4)
      acc = Mfma16<T>::mma(sW[(2 * s + h) * GROUP + mrow], sX[(2 * s + h) * GROUP + mrow], acc);
    __syncthreads();
  };
  chunk(std::integral_constant<int, 0>{});
  if (CT < tiles) chunk(std::integral_constant<int, 1>{});
#pragma unroll
  for (int r = 0; r < 16; r++) red[(wave * 16 + r) * 64 + lane] = acc[r];
  __syncthreads();
  const int rq = wave;                                 // registers 4 * rq .. + 3: four consecutive columns
  const LongType n = n0 + 8 * rq + 4 * h;
  float v[4];
#pragma unroll
  for (int e = 0; e < 4; e++) {
    float sum = 0.f;
#pragma unroll
    for (int w = 0; w < 4; w++) sum += red[(w * 16 + 4 * rq + e) * 64 + lane];
    if (g.bias) sum += to_float(reinterpret_cast<const T*>(g.bias)[n + e]);
    v[e] = sum;
  }
  if (mrow < ROWS && m0 + mrow < g.M) {
    u32x2 o;
    o[0] = (unsigned)Conv<T>::from(v[0]).bits | ((unsigned)Conv<T>::from(v[1]).bits << 16);
    o[1] = (unsigned)Conv<T>::from(v[2]).bits | ((unsigned)Conv<T>::from(v[3]).bits << 16);
    *reinterpret_cast<u32x2*>(C + (m0 + mrow) * g.cRow + n) = o;
    epilogueExtras4<T>(g, m0 + mrow, n, v);
  }
}
template <typename T>
static bool tryGemmSkinny(hipStream_t s, const GemmDesc& d, const void* A, const void* B, void* C) {
  if (d.M < 5 || d.M > 32 || d.batch != 1 || d.alpha != 1.f || d.beta != 0.f) return false;
  if (d.aCol != 1 || d.bRow != 1 || d.cCol != 1) return false;                       // x and Wt k-contiguous, C row-major
  // longer K runs chunk after chunk in one block and measured slower than split-K over many blocks (14 vs 10 us at K = 3072)
  if (d.N % 32 != 0 || d.K % 64 != 0 || d.K > 1024 || d.aRow % 8 != 0 || d.bCol % 8 != 0 || d.cRow % 4 != 0) return false;
  if (((reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(B)) & 15) != 0 || (reinterpret_cast<uintptr_t>(C) & 7) != 0) return false;
  constexpr size_t LDS = (size_t)2 * 6 * 8 * 33 * 16;   // 50,688 B; the 16 KiB of partial tiles reuse it
  static_assert(LDS <= 64 * 1024 && (size_t)4 * 16 * 64 * sizeof(float) <= LDS / 2, "gemm_skinny32 must fit the default dynamic LDS limit");
  GemmArgs g = toArgs(d);
  if (d.lnGain) {
    // what the separate layer_norm runs as one wave per row with one or two 512-value passes: rows of 320 to 768 values
    // with a bias, every vector 16-byte aligned
    if (!d.lnBias || !d.lnOut || d.K < 320 || d.K > 768 || d.lnOutRow % 8 != 0) return false;
    if ((reinterpret_cast<uintptr_t>(d.lnGain) | reinterpret_cast<uintptr_t>(d.lnBias) | reinterpret_cast<uintptr_t>(d.lnOut)) & 15) return false;
    noteKernel("gemm_skinny32<%s,ln>", tname<T>());
    constexpr size_t LDS_LN = LDS + 2 * 128 * 16;          // + gain and bias
    static_assert(LDS_LN <= 64 * 1024, "gemm_skinny32 must fit the default dynamic LDS limit");
    static const bool rows16 = getenv("ND4JHIP_GEMM_SKINNY_ROWS16") ? atoi(getenv("ND4JHIP_GEMM_SKINNY_ROWS16")) != 0 : true;
    // (8 rows per block, 32 threads to a row, measured slower: the batch-32 decode step 0.5215 against 0.5155 ms)
    if (rows16) {
      const dim3 grid((unsigned)(d.N / 32), (unsigned)((d.M + 15) / 16));
      if (d.K <= 512) hipLaunchKernelGGL((gemm_skinny16ln<T, 1>), grid, dim3(256), LDS_LN, s, g, (const T*)A, (const T*)B, (T*)C);
      else hipLaunchKernelGGL((gemm_skinny16ln<T, 2>), grid, dim3(256), LDS_LN, s, g, (const T*)A, (const T*)B, (T*)C);
      return true;
    }
    if (d.K <= 512) hipLaunchKernelGGL((gemm_skinny32<T, 1>), dim3((unsigned)(d.N / 32)), dim3(256), LDS_LN, s, g, (const T*)A, (const T*)B, (T*)C);
    else hipLaunchKernelGGL((gemm_skinny32<T, 2>), dim3((unsigned)(d.N / 32)), dim3(256), LDS_LN, s, g, (const T*)A, (const T*)B, (T*)C);
    return true;
  }
  noteKernel("gemm_skinny32<%s>", tname<T>());
  hipLaunchKernelGGL((gemm_skinny32<T>), dim3((unsigned)(d.N / 32)), dim3(256), LDS, s, g, (const T*)A, (const T*)B, (T*)C);
  return true;
}

// the element-gathering tile kernel: any strides, any alignment (no epilogue outputs, no split-K)
template <typename T, int BM, int BN, int WM, int WN>
static bool launchMfma16uCfg(hipStream_t s, const GemmDesc& d, const void* A, const void* B, void* C) {
  constexpr size_t LDS = (size_t)2 * (TileLayout<BM, true>::SLOTS + TileLayout<BN, true>::SLOTS) * 16;
  const GemmArgs g = toArgs(d);
  auto absl = [](LongType v) { return v < 0 ? -v : v; };
  const bool aRF = absl(d.aRow) < absl(d.aCol), bRF = absl(d.bCol) < absl(d.bRow);   // the smaller stride runs along the rows
  const unsigned tilesM = (unsigned)((d.M + BM - 1) / BM), tilesN = (unsigned)((d.N + BN - 1) / BN);
  const dim3 grid(tilesM * tilesN, 1, (unsigned)d.batch), block(WM * WN * 64);
  noteKernel("gemm_mfma16u<%s,%dx%d,arf=%d,brf=%d>", tname<T>(), BM, BN, (int)aRF, (int)bRF);
#define LAUNCH_U(ARF, BRF) do { \
    if (!DynLds<gemm_mfma16u<T, BM, BN, WM, WN, ARF, BRF>, (int)LDS>::granted()) return false; \
    hipLaunchKernelGGL((gemm_mfma16u<T, BM, BN, WM, WN, ARF, BRF>), grid, block, LDS, s, g, (const T*)A, (const T*)B, (T*)C, tilesM, tilesN); } while (0)
  if (aRF && bRF) LAUNCH_U(true, true); else if (aRF) LAUNCH_U(true, false); else if (bRF) LAUNCH_U(false, true); else LAUNCH_U(false, false);
#undef LAUNCH_U
  return true;
}
template <typename T>
static bool launchMfma16u(hipStream_t s, const GemmDesc& d, const void* A, const void* B, void* C) {
  if (d.M * d.N < 4096 || d.K < 32 || (d.M + 127) / 128 * ((d.N + 127) / 128) >= (1LL << 31)) return false;
  if (d.M <= 32) return launchMfma16uCfg<T, 32, 128, 1, 4>(s, d, A, B, C);
  // (256 x 256 tiles, twice the products per gathered element, measured no faster: 4095^3 720 against 744 us, 2047^3 377 against 202)
  return launchMfma16uCfg<T, 128, 128, 2, 2>(s, d, A, B, C);
}

template <typename T>
static bool dispatch16(hipStream_t s, const GemmDesc& d, const void* A, const void* B, void* C) {
  if (d.attnPartial) {   // only the one-row product against k-contiguous weights merges an attention's parts on the way in
    if (d.M == 1 && d.N > 1 && d.batch == 1 && d.bRow == 1 && d.cCol == 1 && !d.lnGain) return tryGemvRowdotPre<T>(s, d, A, B, C);
    return false;
  }
  if (d.lnGain) {   // only the products of 1 and of 5 to 32 rows against k-contiguous weights normalise their rows on the way in
    if (d.M == 1 && d.N > 1 && d.batch == 1 && d.bRow == 1 && d.cCol == 1) return tryGemvRowdotPre<T>(s, d, A, B, C);
    if (d.M >= 5 && d.M <= 32) return tryGemmSkinny<T>(s, d, A, B, C);
    return false;
  }
  bool aKC = false, bKC = false, aligned = false;
  const bool eligible = (d.M * d.N >= 1024 || (d.M == 1 && d.N >= 64)) && d.K >= 32 && mfmaEligible(d, A, B, sizeof(T), aKC, bKC, aligned);
  // x[1, K] times row-major W[K, N]: the split-K tile kernel streams W with far more loads in flight than the
  // column-sum GEMV (the unused 31 rows of the MFMA tile cost nothing here)
  if (tryGemvStrip<T>(s, d, A, B, C)) return true;
  if (tryGemmSkinny<T>(s, d, A, B, C)) return true;
  const bool rowTimesRowMajor = d.M == 1 && eligible && aKC && !bKC && d.batch == 1;
  if (!rowTimesRowMajor && tryGemv<T>(s, d, A, B, C)) return true;
  if (eligible) {
    GemmArgs g = toArgs(d);
    if (aKC && bKC) return launchMfma16<T, true, true>(s, g, A, B, C, d.batch, aligned);
    if (aKC && !bKC) return launchMfma16<T, true, false>(s, g, A, B, C, d.batch, aligned);
    if (!aKC && bKC) return launchMfma16<T, false, true>(s, g, A, B, C, d.batch, aligned);
    return launchMfma16<T, false, false>(s, g, A, B, C, d.batch, aligned);
  }
  if (d.epi) return false;
  if (launchMfma16u<T>(s, d, A, B, C)) return true;
  launchSimple<T>(s, A, B, C, d);
  return true;
}
static void dispatch32(hipStream_t s, const GemmDesc& d, const void* A, const void* B, void* C) {
  if (tryGemv<float>(s, d, A, B, C)) return;
  bool aKC = false, bKC = false, aligned = false;
  if (d.M * d.N >= 1024 && d.K >= 16 && mfmaEligible(d, A, B, 4, aKC, bKC, aligned)) {
    GemmArgs g = toArgs(d);
    if (aKC && bKC) return launchMfma32<true, true>(s, g, A, B, C, d.batch, aligned);
    if (aKC && !bKC) return launchMfma32<true, false>(s, g, A, B, C, d.batch, aligned);
    if (!aKC && bKC) return launchMfma32<false, true>(s, g, A, B, C, d.batch, aligned);
    return launchMfma32<false, false>(s, g, A, B, C, d.batch, aligned);
  }
  launchSimple<float>(s, A, B, C, d);
}

bool launchGemm(hipStream_t s, DataType dt, const void* A, const void* B, void* C, const GemmDesc& d) {
  if (d.M == 0 || d.N == 0 || d.batch == 0) return true;
  ND4J_REQUIRE(d.batch < 65536 && (d.M + 31) / 32 < 65536 && (d.N + 31) / 32 < (1LL << 31), "matmul: problem too large for the launch grid");
  bool withEpilogue = d.epi != nullptr || d.lnGain != nullptr || d.attnPartial != nullptr;
  if (withEpilogue) {
    // only the 16-bit decode-step kernels carry epilogue outputs; when the dispatch lands elsewhere nothing has been
    // launched yet and the product runs again without the request
    bool done = false;
    if (dt == HALF) done = dispatch16<f16_t>(s, d, A, B, C);
    else if (dt == BFLOAT16) done = dispatch16<bf16_t>(s, d, A, B, C);
    if (done) { HIP_CHECK(hipGetLastError()); return true; }
    if (d.lnGain || d.attnPartial) return false;   // nothing launched: the caller runs the separate op (layer_norm, merge) and calls again
    GemmDesc plain = d;
    plain.epi = nullptr;
    launchGemm(s, dt, A, B, C, plain);
    return false;
  }
  switch (dt) {
    case FLOAT32: dispatch32(s, d, A, B, C); break;
    case DOUBLE: launchSimple<double>(s, A, B, C, d); break;
    case HALF: dispatch16<f16_t>(s, d, A, B, C); break;
    case BFLOAT16: dispatch16<bf16_t>(s, d, A, B, C); break;
    case INT32: case INT64: {
      ND4J_REQUIRE(d.bias == nullptr, "matmul: a bias row with integer arrays is not implemented in nd4j-hip");
      ND4J_REQUIRE(d.M * d.N < (1LL << 39), "matmul: problem too large for the launch grid");
      GemmArgs g = toArgs(d);
      const dim3 grid((unsigned)((d.M * d.N + 255) / 256), 1, (unsigned)d.batch);
      const LongType alphaZ = (LongType)d.alpha, betaZ = (LongType)d.beta;
      if (dt == INT32) { noteKernel("gemm_int<int32>"); hipLaunchKernelGGL((gemm_int<int>), grid, dim3(256), 0, s, g, (const int*)A, (const int*)B, (int*)C, alphaZ, betaZ, d.beta != 0.f ? 1 : 0); }
      else { noteKernel("gemm_int<int64>"); hipLaunchKernelGGL((gemm_int<LongType>), grid, dim3(256), 0, s, g, (const LongType*)A, (const LongType*)B, (LongType*)C, alphaZ, betaZ, d.beta != 0.f ? 1 : 0); }
      break;
    }
    default: ND4J_THROW("matmul: unsupported dtype");
  }
  HIP_CHECK(hipGetLastError());
  return true;
}

}  // namespace nd4jhip
