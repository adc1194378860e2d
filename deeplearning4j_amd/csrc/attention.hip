// Attention kernels for dot_product_attention_v2
// (reference: libnd4j/include/helpers/impl/AttentionHelper.cpp:340-352 logits, :70-79 mask, :189-241 scores).
//
//   attn_fused    - out = softmax(mask(clip(scale * q k^T))) v without materialising anything of size Tq x Tv.
//                   One block = 128 queries of one batch entry (4 waves x 32 queries), looping over 64-key tiles
//                   of K and V that go from global memory straight into LDS (two stages).  The score tile is computed TRANSPOSED, S^T = K Q^T, so that an MFMA
//                   lane owns one query column: the softmax statistics (running max / running sum) and the
//                   rescaling of the output accumulator O^T = V^T P^T are then per-lane scalars, and the row
//                   reductions run over a lane's own registers plus one exchange with the other half-wave.
//                   P^T feeds the second MFMA straight from the score accumulators (the MFMA k-slots are
//                   assigned to keys in exactly the order the accumulator registers hold them, and V^T is read
//                   from LDS in that same order), so the probabilities never leave registers.  The V tile sits in
//                   LDS as it lies in memory ([key][dv]) and is transposed by the read (ds_read_b64_tr_b16).
//                   Logits are rounded through the storage type before the softmax, as the reference's
//                   op-by-op composition stores them in an array of that type.  Masked (key > query) and
//                   out-of-range keys contribute exactly zero; the reference's clamped softmax gives them
//                   e^-88 / sum, below 1e-36.
//                   Bound: MFMA for the contractions, in practice the per-score VALU work (exp, max, convert).
//   logits fix-up - in-place pass over dense [B, Tq, Tv] logits for the composition path that writes the
//                   logits / weights outputs: optional scale, clip to +-1e4, causal penalty.
#include <algorithm>
#include <array>
#include <cmath>
#include <map>
#include <memory>
#include <mutex>
#include <type_traits>

#include "device.h"
#include "kernels.h"
#include "mfma_tile.h"
#include "rowmath.h"
#include "runtime.h"

namespace nd4jhip {

template <typename T>
__global__ __launch_bounds__(256) void logits_fixup(T* __restrict__ l, LongType total, LongType Tq, LongType Tv, float scale,
                                                    int applyScale, int causal, float maskValue, const unsigned char* __restrict__ vmask) {
  const LongType step = (LongType)gridDim.x * 256;
  for (LongType i = (LongType)blockIdx.x * 256 + threadIdx.x; i < total; i += step) {
    const LongType j = i % Tv, r = (i / Tv) % Tq;
    // every step rounds through the storage type, as the reference's op-by-op composition does
    float v = to_float(l[i]);
    if (applyScale) v = to_float(Conv<T>::from(v * to_float(Conv<T>::from(scale))));
    v = v > 1e4f ? to_float(Conv<T>::from(1e4f)) : v;
    v = v < -1e4f ? to_float(Conv<T>::from(-1e4f)) : v;
    // one penalty where the merged mask (causal AND value mask) is false (AttentionHelper.cpp:175-187,199-221)
    bool masked = causal && j > r;
    if (vmask != nullptr && vmask[(i / (Tv * Tq)) * Tv + j] == 0) masked = true;
    if (masked) v = v - maskValue;
    l[i] = Conv<T>::from(v);
  }
}

void launchAttentionLogitsFixup(hipStream_t s, DataType dt, void* logits, const AttnDesc& d) {
  const LongType total = d.B * d.Tq * d.Tv;
  if (total == 0) return;
  LongType blocks = (total + 255) / 256;
  if (blocks > 256 * 16) blocks = 256 * 16;
  dim3 g((unsigned)blocks), b(256);
  switch (dt) {
    case FLOAT32: hipLaunchKernelGGL((logits_fixup<float>), g, b, 0, s, (float*)logits, total, d.Tq, d.Tv, d.scale, (int)d.applyScale, (int)d.causal, d.maskValue, d.vmask); break;
    case HALF: hipLaunchKernelGGL((logits_fixup<f16_t>), g, b, 0, s, (f16_t*)logits, total, d.Tq, d.Tv, d.scale, (int)d.applyScale, (int)d.causal, d.maskValue, d.vmask); break;
    case BFLOAT16: hipLaunchKernelGGL((logits_fixup<bf16_t>), g, b, 0, s, (bf16_t*)logits, total, d.Tq, d.Tv, d.scale, (int)d.applyScale, (int)d.causal, d.maskValue, d.vmask); break;
    default: ND4J_THROW("attention: unsupported dtype");
  }
  HIP_CHECK(hipGetLastError());
}

// weights[b, i, :] *= qmask[b, i], the mask value taken in the weights' type (AttentionHelper.cpp:463-467)
template <typename T>
__global__ __launch_bounds__(256) void weights_query_mask(T* __restrict__ w, LongType total, LongType Tv, const T* __restrict__ qmask) {
  const LongType step = (LongType)gridDim.x * 256;
  for (LongType i = (LongType)blockIdx.x * 256 + threadIdx.x; i < total; i += step)
    w[i] = Conv<T>::from(to_float(w[i]) * to_float(qmask[i / Tv]));
}
void launchAttentionQueryMask(hipStream_t s, DataType dt, void* weights, const void* qmask, const AttnDesc& d) {
  const LongType total = d.B * d.Tq * d.Tv;
  if (total == 0) return;
  LongType blocks = (total + 255) / 256;
  if (blocks > 256 * 16) blocks = 256 * 16;
  dim3 g((unsigned)blocks), b(256);
  switch (dt) {
    case FLOAT32: hipLaunchKernelGGL((weights_query_mask<float>), g, b, 0, s, (float*)weights, total, d.Tv, (const float*)qmask); break;
    case HALF: hipLaunchKernelGGL((weights_query_mask<f16_t>), g, b, 0, s, (f16_t*)weights, total, d.Tv, (const f16_t*)qmask); break;
    case BFLOAT16: hipLaunchKernelGGL((weights_query_mask<bf16_t>), g, b, 0, s, (bf16_t*)weights, total, d.Tv, (const bf16_t*)qmask); break;
    default: ND4J_THROW("attention: unsupported dtype");
  }
  HIP_CHECK(hipGetLastError());
}

// ---- fused kernel ------------------------------------------------------------------------------------------------
struct FusedArgs {
  LongType Tq, Tv;
  LongType qB, qT, kB, kT, vB, vT, oB, oT;
  LongType H, qB2, kB2, vB2, oB2;     // second batch level (H = 0: none)
  float scale;
  int applyScale, causal;
  int qTiles, perBatch, nBatch, heavyFirst;   // fused kernel: work slots per batch entry, batch entries, block order
  const unsigned char* vmask;                 // VM kernels: dense [batch entries, Tv] bytes, 0 = padded key
  float maskValue;                            // what a masked logit has subtracted
  int splits = 1;                             // decode kernel: key ranges per (batch entry, query), blockIdx.z picks one
  float* partial = nullptr;                   // ... and where a range's partial result goes (null: the block writes the output)
};
// Fused kernels, block order 2: block id -> work item (query tile x batch entry, heavy tiles first), a table made on the
// host and passed by value.  Used when every block of the launch is on the chip at once: block ids i, i + 256, i + 512
// then share a CU (the hardware deals consecutive ids out CU after CU and comes round again), and the table gives every
// CU about the same number of key tiles.
constexpr int BLOCK_ORDER_MAX = 768;
struct BlockOrder { unsigned short item[BLOCK_ORDER_MAX]; };

template <typename T> __device__ __forceinline__ float round_storage(float v) { return to_float(Conv<T>::from(v)); }
// round two values through the storage type in place
template <typename T> __device__ __forceinline__ void round_pair(float& a, float& b);
template <> __device__ __forceinline__ void round_pair<bf16_t>(float& a, float& b) {
  const unsigned p = pack_pair<bf16_t>(a, b);
  a = __uint_as_float(p << 16);
  b = __uint_as_float(p & 0xffff0000u);
}
template <> __device__ __forceinline__ void round_pair<f16_t>(float& a, float& b) {
  const f32x2a v = {a, b};
  const f32x2a r = __builtin_convertvector(__builtin_convertvector(v, f16x2a), f32x2a);
  a = r[0]; b = r[1];
}
template <typename T> __device__ __forceinline__ unsigned pack2(float a, float b) {
  return (unsigned)Conv<T>::from(a).bits | ((unsigned)Conv<T>::from(b).bits << 16);
}

// FOLD: the scale is a power of two (or 1) and the scores are bf16, so scaling commutes exactly with the clip and with
// the rounding through the storage type; the kernel then keeps unscaled scores and multiplies inside the exponent's
// fused multiply-add (scale * log2(e) is exact too), which saves one multiply per score.
// VM: a value (padding) mask is present.  Masked logits -- padded keys and, under the causal flag, keys after the query --
// then get the reference's penalty subtracted and rounded through the storage type instead of being dropped, and no key
// tile is skipped: a query whose visible keys are all padded spreads its weight over every key, as the reference's
// softmax over equally penalised logits does.
template <typename T, int D, bool FOLD, bool VM>
__global__ __launch_bounds__(256, D == 64 ? 2 : 1) void attn_fused(FusedArgs a, BlockOrder ord, const T* __restrict__ Q, const T* __restrict__ K, const T* __restrict__ V,
                                                  T* __restrict__ O) {
  constexpr int BQ = 128, BKV = 64, NT = 256;
  constexpr int DG = D / 8;                      // 16-byte groups along d
  constexpr bool OVF = sizeof(T) == 2 && !std::is_same<T, bf16_t>::value;   // fp16: products beyond the type's range
  constexpr int KSLOTS = (D / 64) * 512;         // K tile: 8 chunks of 64 slots (8 keys x 128 bytes) per 64 values of d
  constexpr int VSLOTS = 64 * (D / 8);           // V tile: [key][dv] as in memory, 16-byte slots swizzled inside a key row
  constexpr int DT = D / 32;                     // dv tiles of the output accumulator
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  u32x4* smem = reinterpret_cast<u32x4*>(smem_raw);   // two stages of (K tile, V tile)

  // Two block orders.
  // Batch-major (a.heavyFirst == 0): consecutive block ids go to different XCDs (8 of them, round-robin), so every XCD
  // gets a contiguous run of the (batch entry, work slot) sequence: the query tiles of one batch entry then share that
  // XCD's L2 copy of K and V.  Under the causal mask a block takes a heavy (late) query tile and then its light mirror
  // image, so that every block carries the same number of key tiles (a.perBatch = ceil(qTiles / 2) work slots per
  // batch entry, else qTiles).  Equal blocks waste up to a whole round when they are few per CU.
  // Heavy first (causal mask only; chosen by the host when it pays): block id = query tile (major, last tile first) x
  // batch entry (minor), one query tile per block.  Blocks are handed out in id order as slots on the CUs free up, so
  // the light tiles fill the gaps the heavy ones leave and the CUs finish close together.  With a multiple of 8 batch
  // entries every query tile of an entry still lands on one XCD.
  int slot;
  LongType b;
  if (a.heavyFirst) {
    const unsigned item = a.heavyFirst == 2 ? ord.item[blockIdx.x] : blockIdx.x;   // 2: the host's table (see BlockOrder)
    slot = (int)(item / (unsigned)a.nBatch);
    b = item % (unsigned)a.nBatch;
  } else {
    const unsigned total = gridDim.x, xcd = blockIdx.x & 7u, idx = blockIdx.x >> 3, per = total >> 3, rem = total & 7u;
    const unsigned item = xcd * per + (xcd < rem ? xcd : rem) + idx;
    slot = (int)(item % a.perBatch);
    b = item / a.perBatch;
  }
  if (a.H > 0) {
    const LongType hi = b / a.H, lo = b - hi * a.H;
    Q += hi * a.qB2 + lo * a.qB; K += hi * a.kB2 + lo * a.kB; V += hi * a.vB2 + lo * a.vB; O += hi * a.oB2 + lo * a.oB;
  } else {
    Q += b * a.qB; K += b * a.kB; V += b * a.vB; O += b * a.oB;
  }
  const unsigned char* vm = VM ? a.vmask + b * a.Tv : nullptr;
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6, h = lane >> 5;
  const float sc = a.scale;   // 1 when the op applies no scale
  const float L2E = FOLD ? 1.44269502162933349609375f * sc : 1.44269502162933349609375f;
  const float clip = FOLD ? 1.0e4f / sc : 1.0e4f;
  const unsigned kTb = (unsigned)a.kT * 2u, vTb = (unsigned)a.vT * 2u;   // bytes per key row
  // value tile kept as it lies in memory ([key][dv], 16-byte slots swizzled inside a key row) and read with the transposing
  // LDS read
  using RowV = RowTileLoader<D, NT>;
  // this lane's transposing reads of the value tile, per dv tile of 32: the 16-lane group reads 4 keys x 16 dv; key slot e of
  // k-step ks on half h must be key 16 ks + 8 (e / 4) + 4 h + e % 4 (the order of the score accumulator), so the first read
  // of a k-step starts at key 4 h and the second 8 keys further on
  int trV[D / 32];
#pragma unroll
  for (int i = 0; i < D / 32; i++) {
    const int grp = lane >> 4, i16 = lane & 15;
    const int r4 = i * 32 + 16 * (grp & 1) + 4 * (i16 & 3);
    const int k = 4 * (grp >> 1) + (i16 >> 2);
    trV[i] = (k * RowV::SPR + ((r4 >> 3) ^ RowV::swz(k))) * 16 + ((r4 >> 2) & 1) * 8;
  }
  // Direct loads (global memory -> LDS, no registers): a wave instruction moves one chunk of 1 KiB, 64 slots of 16 bytes in
  // lane order.  K chunk: 8 keys x the 128 bytes of one 64-wide part of d; lane (lj = lane / 8, lp = lane % 8) fetches the
  // k-group that belongs in position lp of key row lj under the XOR placement the fragment reads below undo (the one of the
  // GEMM's k-contiguous operand: conflict-free 16-byte reads by 32 consecutive rows).  V chunk: 64 / SPR keys x one key
  // row of SPR slots, swizzled as RowTileLoader stores them.  Wave w owns chunks w * KPW ... and w * VPW ...
  constexpr int KCH = 8 * (D / 64), VCH = D / 8, KPW = KCH / 4, VPW = VCH / 4;
  const int waveU = __builtin_amdgcn_readfirstlane(wave);
  unsigned dmaK[KPW], dmaKrow[KPW], dmaV[VPW], dmaVrow[VPW];
#pragma unroll
  for (int c = 0; c < KPW; c++) {
    const int ch = waveU * KPW + c, part = ch >> 3, cw = ch & 7, lj = lane >> 3, lp = lane & 7;
    const int lkg = (lp - 4 * (cw & 1) - (lj >> 1)) & 7;
    dmaKrow[c] = (unsigned)(8 * cw + lj);
    dmaK[c] = (unsigned)(part * 128 + lkg * 16);
  }
#pragma unroll
  for (int c = 0; c < VPW; c++) {
    const int ch = waveU * VPW + c, k = ch * (64 / RowV::SPR) + lane / RowV::SPR, pp = lane % RowV::SPR;
    dmaVrow[c] = (unsigned)k;
    dmaV[c] = (unsigned)((pp ^ RowV::swz(k)) * 16);
  }
  const bool paired = !a.heavyFirst && a.perBatch != a.qTiles;
  for (int pass = 0; pass < (paired ? 2 : 1); pass++) {
  const int qt = pass == 0 ? a.qTiles - 1 - slot : slot;
  if (pass == 1 && qt >= a.qTiles - 1 - slot) break;   // odd count: the middle tile has no mirror image
  const LongType q0 = (LongType)qt * BQ;
  const LongType query = q0 + wave * 32 + (lane & 31);
  const LongType qrow = query < a.Tq ? query : a.Tq - 1;

  // Q^T fragments: lane (query, h) holds d = 16*ks + 8*h .. +7 for every k-step
  u32x4 qf[D / 16];
#pragma unroll
  for (int ks = 0; ks < D / 16; ks++) qf[ks] = *reinterpret_cast<const u32x4*>(Q + qrow * a.qT + ks * 16 + h * 8);

  f32x16 o[DT];
#pragma unroll
  for (int i = 0; i < DT; i++)
#pragma unroll
    for (int r = 0; r < 16; r++) o[i][r] = 0.f;
  float m = -1.0e30f, l = 0.f;

  LongType kvEnd = a.Tv;
  if (a.causal && !VM) { const LongType lim = q0 + BQ; kvEnd = lim < kvEnd ? lim : kvEnd; }
  const LongType nTiles = (kvEnd + BKV - 1) / BKV;

  typedef __attribute__((address_space(3))) void* lds_ptr;
  // written as assembly so that the compiler's wait-count pass does not know of an outstanding write into LDS (it would
  // wait for these loads in front of every transposing LDS read); all waiting for them is explicit, in front of the
  // barrier that ends a key tile.  M0 carries the LDS address of the chunk; nothing else in this kernel uses M0.
  // address = scalar base (the tile's first key row, the same for every lane) + 32-bit lane offset: no vector arithmetic
  auto dma = [&](const char* base, unsigned off, const u32x4* dst) {
    const unsigned ldsAddr = (unsigned)(size_t)(lds_ptr)dst;
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(off), "s"(base), "s"(ldsAddr) : "memory");
  };
  unsigned fullK[KPW], fullV[VPW];   // lane offsets inside a whole tile
#pragma unroll
  for (int c = 0; c < KPW; c++) fullK[c] = dmaKrow[c] * kTb + dmaK[c];
#pragma unroll
  for (int c = 0; c < VPW; c++) fullV[c] = dmaVrow[c] * vTb + dmaV[c];
  auto issueKV = [&](LongType kv0, u32x4* stage) {
    const char* kt = reinterpret_cast<const char*>(K + kv0 * a.kT);
    const char* vt = reinterpret_cast<const char*>(V + kv0 * a.vT);
    if (kv0 + BKV <= a.Tv) {
#pragma unroll
      for (int c = 0; c < KPW; c++) dma(kt, fullK[c], stage + (waveU * KPW + c) * 64);
#pragma unroll
      for (int c = 0; c < VPW; c++) dma(vt, fullV[c], stage + KSLOTS + (waveU * VPW + c) * 64);
    } else {
      // the last, ragged tile: keys past the end repeat the last one (their weights are exactly 0)
      const unsigned last = (unsigned)(a.Tv - 1 - kv0);
#pragma unroll
      for (int c = 0; c < KPW; c++) {
        const unsigned row = dmaKrow[c] < last ? dmaKrow[c] : last;
        dma(kt, row * kTb + dmaK[c], stage + (waveU * KPW + c) * 64);
      }
#pragma unroll
      for (int c = 0; c < VPW; c++) {
        const unsigned row = dmaVrow[c] < last ? dmaVrow[c] : last;
        dma(vt, row * vTb + dmaV[c], stage + KSLOTS + (waveU * VPW + c) * 64);
      }
    }
  };
  // this lane's K fragment slots: key row r = 32 kt + lane % 32, k-group 2 ks + h of part ks / 4
  auto slotK = [&](int kg, int r) {
    return (kg >> 3) * 512 + (r >> 3) * 64 + 8 * (r & 7) + (((kg & 7) + 4 * ((r >> 3) & 1) + ((r & 7) >> 1)) & 7);
  };
  if (nTiles > 0) issueKV(0, smem);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  // Make the Q fragments "used" here, on every path into the key loop: otherwise the path that skips the block above
  // leaves their loads pending as far as the compiler can tell, and it waits for them -- and with them for the freshly
  // issued loads of the next tile -- in front of the first MFMAs of every iteration.
#pragma unroll
  for (int ks = 0; ks < D / 16; ks++) asm volatile("" : "+v"(qf[ks]));

  for (LongType it = 0; it < nTiles; it++) {
    const int cur = (int)(it & 1);
    const LongType kv0 = it * BKV;
    const u32x4* sK = smem + cur * (KSLOTS + VSLOTS);
    const u32x4* sV = sK + KSLOTS;
    const bool more = it + 1 < nTiles;
    if (more) issueKV(kv0 + BKV, smem + (cur ^ 1) * (KSLOTS + VSLOTS));   // lands in the other stage while this tile is computed

    // S^T = K Q^T : two 32-key tiles, D/16 k-steps
    f32x16 s[2];
#pragma unroll
    for (int kt = 0; kt < 2; kt++) {
#pragma unroll
      for (int r = 0; r < 16; r++) s[kt][r] = 0.f;
#pragma unroll
      for (int ks = 0; ks < D / 16; ks++) {
        const u32x4 kf = sK[slotK(ks * 2 + h, kt * 32 + (lane & 31))];   // parts of 8 k-groups follow each other
        s[kt] = Mfma16<T>::mma(kf, qf[ks], s[kt]);
      }
    }
    // The softmax arithmetic below runs at raised wave priority, the MFMA sections and the tile store at the normal one:
    // of the two waves that share a SIMD the one in its vector phase then gets the issue slots it is bound by, while the
    // other's MFMAs, which only need a slot every 32 cycles, fill in (33.0 against 34.5 us on [96, 1024, 64] causal).
    __builtin_amdgcn_s_setprio(1);
    // scores of this lane's query: register r of tile kt is key kv0 + 32*kt + 8*(r/4) + 4*h + r%4.
    // scale, clip to +-1e4, round through the storage type (two scores per conversion).  The clip is one instruction per
    // score that almost never changes anything, so tiles without masked entries first take the maximum of the raw scores:
    // scaling by a positive factor, clipping and rounding are monotonic, so the tile's maximum after all three is the
    // three applied to that one value, and when it does not exceed the clip no score does.  At the lower end a score below
    // -clip and its clipped value both give an exponential of exactly 0 once the running maximum lies 160 / log2(e)
    // above -clip.  Only when a wave fails one of the two tests (or the scale is not positive) does it clip every score.
    const int qFirst = (int)q0 + wave * 32;
    const bool maskedTile = VM || __builtin_amdgcn_readfirstlane((int)((a.causal && (int)kv0 + BKV - 1 > qFirst) || kv0 + BKV > a.Tv)) != 0;
    float tmax = m;
    bool clipAll = true;
    if (!maskedTile) {
      float rmax = s[0][0];
#pragma unroll
      for (int kt = 0; kt < 2; kt++)
#pragma unroll
        for (int r = 0; r < 16; r++) rmax = __builtin_fmaxf(rmax, s[kt][r]);
      const float smax = FOLD ? rmax : rmax * sc;
      tmax = __builtin_fmaxf(m, round_storage<T>(__builtin_amdgcn_fmed3f(smax, -clip, clip)));
      tmax = __builtin_fmaxf(tmax, __shfl_xor(tmax, 32, WAVE));
      // fp16: the reference's logits array holds the raw product in fp16, +-inf beyond 65504 (65520 with rounding), which
      // scaling leaves and the clip turns into +-1e4 -- a tile with such a product is clipped score by score, with the
      // overflow restated; at the lower end the same zero-exponential argument holds from -65520 * scale on
      const float lowest = OVF && 65520.f * sc < clip ? 65520.f * sc : clip;
      const bool fast = sc > 0.f && smax <= clip && (!OVF || rmax < 65520.f) && tmax >= 160.f / L2E - lowest;
      clipAll = __builtin_amdgcn_ballot_w64(!fast) != 0;
    }
    // (the clip works on the registers in place and the rounding below is common to both cases: written as two complete
    // alternatives the compiler merged them with 32 register copies per tile)
    if (clipAll) {
      asm volatile("; scores clipped one by one");
#pragma unroll
      for (int kt = 0; kt < 2; kt++)
#pragma unroll
        for (int r = 0; r < 16; r++) {
          float v = s[kt][r];
          if (OVF) v = __builtin_fabsf(v) >= 65520.f ? __builtin_copysignf(__builtin_inff(), v) : v;
          if (!FOLD) v *= sc;
          s[kt][r] = __builtin_amdgcn_fmed3f(v, -clip, clip);
        }
    } else if (!FOLD) {
#pragma unroll
      for (int kt = 0; kt < 2; kt++)
#pragma unroll
        for (int r = 0; r < 16; r++) s[kt][r] *= sc;
    }
#pragma unroll
    for (int kt = 0; kt < 2; kt++)
#pragma unroll
      for (int r = 0; r < 16; r += 2) {
        float v0 = s[kt][r], v1 = s[kt][r + 1];
        round_pair<T>(v0, v1);
        s[kt][r] = v0; s[kt][r + 1] = v1;
      }
    // only tiles that touch the diagonal or the end of the keys carry masked entries (wave-uniform test)
    // a real branch (scalar condition, a body the compiler cannot speculate): turned into selects, the mask costs 86
    // vector instructions on every tile instead of on the few that need it
    if (VM) {
      const int lastVisible = a.causal ? (int)query : (int)a.Tv - 1;
#pragma unroll
      for (int kt = 0; kt < 2; kt++)
#pragma unroll
        for (int r4 = 0; r4 < 4; r4++) {
          const int key0 = (int)kv0 + kt * 32 + 8 * r4 + 4 * h;   // registers 4*r4 .. +3 hold four consecutive keys
#pragma unroll
          for (int e = 0; e < 4; e++) {
            const int key = key0 + e;
            const float sv = s[kt][4 * r4 + e];
            if (key >= (int)a.Tv) s[kt][4 * r4 + e] = -1.0e30f;    // beyond the keys: contributes exactly nothing
            else if (key > lastVisible || vm[key] == 0) s[kt][4 * r4 + e] = round_storage<T>(sv - a.maskValue);
          }
        }
    } else if (maskedTile) {
      asm volatile("; tile with masked entries");
      const int lastKey = a.causal ? ((int)query < (int)a.Tv - 1 ? (int)query : (int)a.Tv - 1) : (int)a.Tv - 1;
#pragma unroll
      for (int kt = 0; kt < 2; kt++)
#pragma unroll
        for (int r = 0; r < 16; r++) {
          const int key = (int)kv0 + kt * 32 + 8 * (r / 4) + 4 * h + (r & 3);
          s[kt][r] = key > lastKey ? -1.0e30f : s[kt][r];
        }
    }
    if (maskedTile) {   // the maximum of what is left after masking
#pragma unroll
      for (int kt = 0; kt < 2; kt++)
#pragma unroll
        for (int r = 0; r < 16; r++) tmax = __builtin_fmaxf(tmax, s[kt][r]);
      tmax = __builtin_fmaxf(tmax, __shfl_xor(tmax, 32, WAVE));
    }
    // every query has seen key 0 by now, so the running maximum is a real score and masked entries (-1e30)
    // underflow to exactly 0 in the exponential
    const float mL = tmax * L2E;
    // With a value mask a query may have seen nothing but hidden keys so far (fp16: their logits are -inf), so m and
    // tmax may both still be the -1e30 start value: the difference is taken first, which is exactly 0 then, where the
    // fused form below would turn the rounding error of -1e30 * log2(e) into a factor of 0 or inf.
    const float alpha = VM ? __builtin_amdgcn_exp2f((m - tmax) * L2E) : __builtin_amdgcn_exp2f(m * L2E - mL);
    m = tmax;
    float psum = 0.f;
    u32x4 pf[4];   // P^T operand of k-step ks: registers 8*(ks%2) .. +7 of tile ks/2
#pragma unroll
    for (int kt = 0; kt < 2; kt++)
#pragma unroll
      for (int r = 0; r < 16; r += 2) {
        float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[kt][r], L2E, -mL));
        float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[kt][r + 1], L2E, -mL));
        pf[kt * 2 + r / 8][(r % 8) / 2] = pack_pair<T>(p0, p1);
        psum += p0 + p1;
      }
    l = l * alpha + psum;
    // the accumulator only needs rescaling when some query's maximum moved
    if (__builtin_amdgcn_ballot_w64(alpha != 1.f) != 0) {
      asm volatile("; accumulator rescale");   // keeps this a branch: most tiles leave every maximum where it was
#pragma unroll
      for (int i = 0; i < DT; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) o[i][r] *= alpha;
    }

    // O^T += V^T P^T : k-slot e of k-step ks on half h is key 16*ks + 8*(e/4) + 4*h + e%4 (the accumulator order)
    __builtin_amdgcn_s_setprio(0);
#pragma unroll
    for (int ks = 0; ks < 4; ks++) {
#pragma unroll
      for (int i = 0; i < DT; i++) {
        typedef __attribute__((address_space(3))) void* lds_ptr;
        typedef short s16x4 __attribute__((ext_vector_type(4)));
        const __attribute__((address_space(3))) unsigned char* base =
            (const __attribute__((address_space(3))) unsigned char*)(lds_ptr)sV + trV[i] + ks * (16 * RowV::SPR * 16);
        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)base);
        const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(base + 8 * RowV::SPR * 16));
        const u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
        const u32x4 vf = {l2[0], l2[1], h2[0], h2[1]};
        o[i] = Mfma16<T>::mma(vf, pf[ks], o[i]);
      }
    }
    // nothing that consumes the next tile's registers may drift up into the MFMA sections: the wait for those loads belongs
    // here, after a whole tile of work
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // this wave's chunks of the next tile have landed
    __syncthreads();
  }

  // normalise and write O: register r of dv-tile i is dv = 32*i + 8*(r/4) + 4*h + r%4
  l += __shfl_xor(l, 32, WAVE);
  const float inv = l > 0.f ? 1.f / l : 0.f;
  if (query < a.Tq) {
    T* orow = O + query * a.oT;
#pragma unroll
    for (int i = 0; i < DT; i++)
#pragma unroll
      for (int r4 = 0; r4 < 4; r4++) {
        const int dv = i * 32 + 8 * r4 + 4 * h;
        u32x2 w;
        w[0] = pack2<T>(o[i][4 * r4] * inv, o[i][4 * r4 + 1] * inv);
        w[1] = pack2<T>(o[i][4 * r4 + 2] * inv, o[i][4 * r4 + 3] * inv);
        *reinterpret_cast<u32x2*>(orow + dv) = w;
      }
  }
  }   // pass
}

// ---- decode kernel -------------------------------------------------------------------------------------------------
// A handful of query rows against a long key/value history (Tq <= 8, no causal mask): the work is streaming K and V
// once, so it runs on the vector ALU with 16-byte loads.  One block per (batch entry, query); a key row is covered by
// D/8 neighbouring lanes (8 values of d each), so a wave reads 64 / (D/8) whole rows per load instruction.  The dot
// product is finished with a butterfly over those lanes, which leaves the score in every lane of the key's group --
// exactly where the P V accumulation needs it.  Each lane group keeps its own running (max, sum, o[8]) state;
// states are merged across groups (shuffles), across waves (LDS) and normalised once.  Logits go through the same
// scale / clip / storage-type rounding as in the tile kernel above; probabilities stay in fp32.
// eight consecutive values of d as a lane holds them: one 16-byte load for the 16-bit types, two for fp32
template <typename T> struct Row8 {
  using raw = typename RawIO<T>::raw;
  template <bool NT = false>
  static __device__ __forceinline__ raw load(const T* p) {
    if constexpr (NT) return __builtin_nontemporal_load(reinterpret_cast<const raw*>(p));
    else return *reinterpret_cast<const raw*>(p);
  }
  static __device__ __forceinline__ void unpack(const raw& r, float* out) { RawIO<T>::unpack(r, out); }
};
template <> struct Row8<float> {
  struct raw { raw_f32x4 lo, hi; };
  template <bool NT = false>
  static __device__ __forceinline__ raw load(const float* p) {
    raw r;
    if constexpr (NT) {
      r.lo = __builtin_nontemporal_load(reinterpret_cast<const raw_f32x4*>(p));
      r.hi = __builtin_nontemporal_load(reinterpret_cast<const raw_f32x4*>(p + 4));
    } else {
      r.lo = *reinterpret_cast<const raw_f32x4*>(p);
      r.hi = *reinterpret_cast<const raw_f32x4*>(p + 4);
    }
    return r;
  }
  static __device__ __forceinline__ void unpack(const raw& r, float* out) {
#pragma unroll
    for (int e = 0; e < 4; e++) { out[e] = r.lo[e]; out[4 + e] = r.hi[e]; }
  }
};
// STREAM: keys and values come through non-temporal loads -- a history that is large against the last-level cache (a
// decode step at batch 32 reads 57 MB of it per layer, 680 MB per step) then does not push the weights out of it
template <typename T, int D, int NW, bool VM, int U = 4, bool STREAM = false>
__global__ __launch_bounds__(NW * 64) void attn_decode(FusedArgs a, const T* __restrict__ Q, const T* __restrict__ K, const T* __restrict__ V,
                                                       T* __restrict__ O) {
  constexpr int CH = D / 8;          // lanes per key row
  constexpr int KPS = 64 / CH;       // key rows per load instruction
  // U: load instructions in flight per operand and wave (8, which covers a 1024-key history in one trip to memory when 16
  // waves share it, measured slower than 4: 0.36 against 0.34 ms per decode step)
  __shared__ float sm[NW][D + 2];
  __shared__ __attribute__((aligned(16))) float so[NW][64 / (D / 8)][D];   // per wave: one partial output row per lane group
  typedef __attribute__((ext_vector_type(4))) float f32x4s;
  const LongType b = blockIdx.x, qi = blockIdx.y;
  if (a.H > 0) {
    const LongType hi = b / a.H, lo = b - hi * a.H;
    Q += hi * a.qB2 + lo * a.qB; K += hi * a.kB2 + lo * a.kB; V += hi * a.vB2 + lo * a.vB; O += hi * a.oB2 + lo * a.oB;
  } else {
    Q += b * a.qB; K += b * a.kB; V += b * a.vB; O += b * a.oB;
  }
  const unsigned char* vm = VM ? a.vmask + b * a.Tv : nullptr;
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int g = lane / CH, c = lane % CH;
  // the query row was written by the kernel before this one and the first keys come cold from HBM: all of these loads
  // are issued before the first value is touched, so the two latencies overlap
  using Raw = typename Row8<T>::raw;
  const Raw qraw = Row8<T>::load(Q + qi * a.qT + c * 8);
  // this block's key range (the whole history unless it is cut up)
  LongType kBeg = 0, kEnd = a.Tv;
  if (a.splits > 1) {
    const LongType per = (a.Tv + a.splits - 1) / a.splits;
    kBeg = (LongType)blockIdx.z * per;
    kEnd = kBeg + per < a.Tv ? kBeg + per : a.Tv;
    if (kBeg > kEnd) kBeg = kEnd;
  }
  // (a second register set, so that the next trip's loads fly while the current one is consumed, changed nothing at
  // batch 1 and cost 1 % at batch 32: a block's stream is bound by what one CU can pull, not by a trip's latency)
  Raw krA[U], vrA[U];
  bool validA[U];
  auto issue = [&](LongType k0, Raw (&kr)[U], Raw (&vr)[U], bool (&valid)[U]) {
#pragma unroll
    for (int u = 0; u < U; u++) {
      LongType key = k0 + u * KPS + g;
      valid[u] = key < kEnd;
      key = valid[u] ? key : a.Tv - 1;
      kr[u] = Row8<T>::template load<STREAM>(K + key * a.kT + c * 8);
      vr[u] = Row8<T>::template load<STREAM>(V + key * a.vT + c * 8);
    }
  };
  const LongType step = (LongType)NW * (KPS * U);
  LongType k0 = kBeg + (LongType)wave * (KPS * U);
  if (k0 < kEnd) issue(k0, krA, vrA, validA);
  float q[8];
  Row8<T>::unpack(qraw, q);
  const float L2E = 1.44269502162933349609375f;
  float m = -1.0e30f, l = 0.f, o[8];
#pragma unroll
  for (int e = 0; e < 8; e++) o[e] = 0.f;

  auto consume = [&](LongType k0, const Raw (&kr)[U], const Raw (&vr)[U], const bool (&valid)[U]) {
    float sc[U], tmax = m;
#pragma unroll
    for (int u = 0; u < U; u++) {
      float kf[8];
      Row8<T>::unpack(kr[u], kf);
      float d = 0.f;
#pragma unroll
      for (int e = 0; e < 8; e++) d = __builtin_fmaf(q[e], kf[e], d);
      // butterfly over the CH lanes of the key row, one DPP add per level (the same pairs in the same order as an
      // exchange with lane ^ 1, ^ 2, ^ 4, ^ 8: after two levels a quad holds one value, so a mirror is an exchange)
      d += dpp_f<0xB1>(d);                 // quad_perm [1,0,3,2]
      d += dpp_f<0x4E>(d);                 // quad_perm [2,3,0,1]
      d += dpp_f<0x141>(d);                // row_half_mirror
      if (CH > 8) d += dpp_f<0x140>(d);    // row_mirror
      d = round_storage<T>(d);             // the product as the reference's logits array stores it (fp16: +-inf beyond its range)
      if (a.applyScale) d *= a.scale;
      d = __builtin_fminf(__builtin_fmaxf(d, -1.0e4f), 1.0e4f);
      d = round_storage<T>(d);
      if (VM) {   // a padded key keeps its logit, penalised and rounded as the reference stores it
        const LongType key = k0 + u * KPS + g;
        if (valid[u] && vm[key] == 0) d = round_storage<T>(d - a.maskValue);
      }
      sc[u] = valid[u] ? d : -1.0e30f;
      tmax = __builtin_fmaxf(tmax, sc[u]);
    }
    const float alpha = __builtin_amdgcn_exp2f((m - tmax) * L2E);
    m = tmax;
    l *= alpha;
#pragma unroll
    for (int e = 0; e < 8; e++) o[e] *= alpha;
#pragma unroll
    for (int u = 0; u < U; u++) {
      const float p = valid[u] ? __builtin_amdgcn_exp2f((sc[u] - m) * L2E) : 0.f;
      float vf[8];
      Row8<T>::unpack(vr[u], vf);
      l += p;
#pragma unroll
      for (int e = 0; e < 8; e++) o[e] = __builtin_fmaf(p, vf[e], o[e]);
    }
  };
  while (k0 < kEnd) {
    consume(k0, krA, vrA, validA);
    k0 += step;
    if (k0 < kEnd) issue(k0, krA, vrA, validA);
  }
  // merge the lane groups of the wave (lanes with equal c): bring every state to the wave's maximum, then add.  Max and
  // sum of l run on DPP; the eight-float partial rows go through the wave's own LDS region, where lane d sums element d
  // of every group -- exchanging them lane to lane instead (nine values, three levels of cross-lane permutes per wave)
  // kept the LDS crossbar of the one CU a sixteen-wave block runs on busy for 2 us, half the kernel.
  constexpr int G = 64 / CH;   // lane groups per wave
  const float mAll = wave_allreduce<MaxOp>(m);
  const float f = __builtin_amdgcn_exp2f((m - mAll) * L2E);
  // the CH lanes of a group hold one l: the wave sum counts it CH times (a power of two, so the division is exact)
  const float lAll = wave_allreduce<SumOp>(l * f) * (1.0f / CH);
  {
    float* mine = &so[wave][g][c * 8];
    *reinterpret_cast<f32x4s*>(mine) = f32x4s{o[0] * f, o[1] * f, o[2] * f, o[3] * f};
    *reinterpret_cast<f32x4s*>(mine + 4) = f32x4s{o[4] * f, o[5] * f, o[6] * f, o[7] * f};
  }
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the wave reads what its own lanes wrote: no barrier needed
#pragma unroll
  for (int part = 0; part < D / 64; part++) {
    float acc = 0.f;
#pragma unroll
    for (int gg = 0; gg < G; gg++) acc += so[wave][gg][part * 64 + lane];
    sm[wave][part * 64 + lane] = acc;
  }
  if (lane == 0) { sm[wave][D] = mAll; sm[wave][D + 1] = lAll; }
  __syncthreads();
  if (t < D) {
    float mm = -1.0e30f;
#pragma unroll
    for (int w = 0; w < NW; w++) mm = __builtin_fmaxf(mm, sm[w][D]);
    float lt = 0.f, ot = 0.f;
#pragma unroll
    for (int w = 0; w < NW; w++) {
      const float fw = __builtin_amdgcn_exp2f((sm[w][D] - mm) * L2E);
      lt = __builtin_fmaf(sm[w][D + 1], fw, lt);
      ot = __builtin_fmaf(sm[w][t], fw, ot);
    }
    if (a.partial) {
      // one key range of several: the sums stay relative to this range's maximum; whoever merges the ranges normalises
      float* P = a.partial + ((b * a.Tq + qi) * a.splits + blockIdx.z) * ATTN_PART_PITCH(D);
      P[t] = ot;
      if (t == 0) { P[D] = mm; P[D + 1] = lt; }
    } else {
      O[qi * a.oT + t] = Conv<T>::from(lt > 0.f ? ot / lt : 0.f);
    }
  }
}
// the output rows from the partial results of the key ranges: one block per (batch entry, query), a thread per element
template <typename T, int D>
__global__ __launch_bounds__(D) void attn_merge(FusedArgs a, T* __restrict__ O) {
  const LongType b = blockIdx.x, qi = blockIdx.y;
  if (a.H > 0) {
    const LongType hi = b / a.H, lo = b - hi * a.H;
    O += hi * a.oB2 + lo * a.oB;
  } else {
    O += b * a.oB;
  }
  float v[1];
  attn_merge_vec<1>(a.partial + (b * a.Tq + qi) * a.splits * ATTN_PART_PITCH(D), a.splits, D, (int)threadIdx.x, v);
  O[qi * a.oT + threadIdx.x] = Conv<T>::from(v[0]);
}

// One query token against a long history (a decode step at batch 1: one block per head, whose keys and values all come
// through one CU): cut the history into ranges of at least 128 keys so that about 48 blocks share the read.  Only where the
// heads of that one token are the whole problem: the merge of the ranges is then a step the one-row product that consumes
// the output can take in (a recorded sequence does that); with more rows it would stay a launch of its own, which costs more
// than the cut saves.
int attentionDecodeSplits(const AttnDesc& d) {
  const bool oneToken = d.Tq == 1 && (d.H > 0 ? d.B == d.H : d.B == 1);
  if (!oneToken || d.vmask != nullptr || d.B > 24 || d.Tv < 256) return 1;
  LongType s = 48 / (d.B * d.Tq);
  if (s > d.Tv / 128) s = d.Tv / 128;
  return s >= 8 ? 8 : s >= 4 ? 4 : s >= 2 ? 2 : 1;   // (the merge routines are built for 2, 4 and 8 parts)
}

bool attentionDecodeSupported(DataType dt, const AttnDesc& d) {
  if (dt != HALF && dt != BFLOAT16 && dt != FLOAT32) return false;
  if (d.D != d.Dv || (d.D != 64 && d.D != 128)) return false;
  if (d.causal || d.Tq < 1 || d.Tq > 8 || d.Tv < 1) return false;
  const LongType perVector = dt == FLOAT32 ? 4 : 8;   // rows start on 16-byte boundaries
  for (LongType st : {d.qB, d.qT, d.kB, d.kT, d.vB, d.vT, d.qB2, d.kB2, d.vB2}) if (st % perVector != 0) return false;
  return d.B < (1LL << 31);
}

template <typename T, int D>
static void launchDecodeTyped(hipStream_t s, const void* q, const void* k, const void* v, void* out, const AttnDesc& d) {
  FusedArgs a;
  a.Tq = d.Tq; a.Tv = d.Tv;
  a.qB = d.qB; a.qT = d.qT; a.kB = d.kB; a.kT = d.kT; a.vB = d.vB; a.vT = d.vT; a.oB = d.oB; a.oT = d.oT;
  a.H = d.H; a.qB2 = d.qB2; a.kB2 = d.kB2; a.vB2 = d.vB2; a.oB2 = d.oB2;
  a.scale = d.scale; a.applyScale = d.applyScale ? 1 : 0; a.causal = 0; a.qTiles = 1; a.perBatch = 1;
  a.vmask = d.vmask; a.maskValue = d.maskValue;
  a.splits = 1; a.partial = nullptr;
  if (d.splits > 1) {
    // a range per block (8 waves: a range of a few hundred keys is one trip to memory), then the merge unless the caller
    // leaves it to its next kernel
    ND4J_REQUIRE(d.partial != nullptr && d.vmask == nullptr, "attention: the cut-up decode kernel needs a partial buffer and takes no value mask");
    a.splits = d.splits; a.partial = d.partial;
    hipLaunchKernelGGL((attn_decode<T, D, 8, false>), dim3((unsigned)d.B, (unsigned)d.Tq, (unsigned)d.splits), dim3(512), 0, s, a, (const T*)q, (const T*)k,
                       (const T*)v, (T*)out);
    if (!d.mergeLater) hipLaunchKernelGGL((attn_merge<T, D>), dim3((unsigned)d.B, (unsigned)d.Tq), dim3(D), 0, s, a, (T*)out);
    return;
  }
  const dim3 grid((unsigned)d.B, (unsigned)d.Tq);
  if (d.vmask) {
    hipLaunchKernelGGL((attn_decode<T, D, 4, true>), grid, dim3(256), 0, s, a, (const T*)q, (const T*)k, (const T*)v, (T*)out);
    return;
  }
  // few (batch, head) rows: more waves per row, so that the history is still spread over many loads in flight
  if (d.B * d.Tq < 128) hipLaunchKernelGGL((attn_decode<T, D, 16, false>), grid, dim3(1024), 0, s, a, (const T*)q, (const T*)k, (const T*)v, (T*)out);
  else if ((double)d.B * (double)d.Tv * 2.0 * D * sizeof(T) >= (double)(32 << 20))
    hipLaunchKernelGGL((attn_decode<T, D, 4, false, 4, true>), grid, dim3(256), 0, s, a, (const T*)q, (const T*)k, (const T*)v, (T*)out);
  else hipLaunchKernelGGL((attn_decode<T, D, 4, false>), grid, dim3(256), 0, s, a, (const T*)q, (const T*)k, (const T*)v, (T*)out);
}

template <typename T, int D>
static void launchMergeTyped(hipStream_t s, void* out, const AttnDesc& d) {
  FusedArgs a;
  a.Tq = d.Tq; a.Tv = d.Tv; a.oB = d.oB; a.oT = d.oT; a.H = d.H; a.oB2 = d.oB2;
  a.splits = d.splits; a.partial = d.partial;
  hipLaunchKernelGGL((attn_merge<T, D>), dim3((unsigned)d.B, (unsigned)d.Tq), dim3(D), 0, s, a, (T*)out);
}
void launchAttentionDecodeMerge(hipStream_t s, DataType dt, void* out, const AttnDesc& d) {
  ND4J_REQUIRE(d.splits > 1 && d.partial != nullptr && (d.D == 64 || d.D == 128), "attention: nothing to merge");
  if (dt == HALF) { if (d.D == 64) launchMergeTyped<f16_t, 64>(s, out, d); else launchMergeTyped<f16_t, 128>(s, out, d); }
  else if (dt == BFLOAT16) { if (d.D == 64) launchMergeTyped<bf16_t, 64>(s, out, d); else launchMergeTyped<bf16_t, 128>(s, out, d); }
  else { if (d.D == 64) launchMergeTyped<float, 64>(s, out, d); else launchMergeTyped<float, 128>(s, out, d); }
  HIP_CHECK(hipGetLastError());
}
void launchAttentionDecode(hipStream_t s, DataType dt, const void* q, const void* k, const void* v, void* out, const AttnDesc& d) {
  ND4J_REQUIRE(attentionDecodeSupported(dt, d), "attention: decode kernel does not take this problem");
  ND4J_REQUIRE((((uintptr_t)q | (uintptr_t)k | (uintptr_t)v) & 15) == 0, "attention: operands must be 16-byte aligned");
  if (dt == HALF) { if (d.D == 64) launchDecodeTyped<f16_t, 64>(s, q, k, v, out, d); else launchDecodeTyped<f16_t, 128>(s, q, k, v, out, d); }
  else if (dt == FLOAT32) { if (d.D == 64) launchDecodeTyped<float, 64>(s, q, k, v, out, d); else launchDecodeTyped<float, 128>(s, q, k, v, out, d); }
  else { if (d.D == 64) launchDecodeTyped<bf16_t, 64>(s, q, k, v, out, d); else launchDecodeTyped<bf16_t, 128>(s, q, k, v, out, d); }
  HIP_CHECK(hipGetLastError());
}


// ---- fused kernel, fp32 ------------------------------------------------------------------------------------------------
// The same formulation on the fp32 matrix instruction (v_mfma_f32_32x32x2_f32: a 32 x 32 tile, two k per issue, 64 cycles):
// one block = 128 queries of one batch entry (4 waves x 32 queries), 32-key tiles of K and V staged through LDS in two
// stages (global -> registers -> LDS: at 64 cycles per MFMA the matrix pipe, not the staging, sets the pace).
// S^T = K Q^T: the k index of an MFMA step may be any permutation as long as both operands agree, so the half-wave h takes
// d = h * D/2 + step; a lane then reads its key row's d-range as 16-byte vectors and keeps its query's d-range in registers.
// Lane (query = lane % 32, h) ends up with the scores of keys 8 (r / 4) + 4 h + r % 4, r = 0..15, of its own query: the
// running maximum and sum are per-lane scalars shared with the other half-wave by one exchange, and the probabilities feed
// O^T = V^T P^T straight from those registers (step r of the second product pairs register r of both half-waves).
// Scores are scale * q.k clipped to +-1e4 (AttentionHelper.cpp:340-352); masked and out-of-range keys weigh exactly 0
// (the reference's clamped softmax gives them e^-88 / sum).  No value mask here: such calls take the composition.
template <int D>
__global__ __launch_bounds__(256, D == 64 ? 3 : 1) void attn_fused_f32(FusedArgs a, BlockOrder ord, const float* __restrict__ Q, const float* __restrict__ K, const float* __restrict__ V,
                                                      float* __restrict__ O) {
  constexpr int BQ = 128, BKV = 32, HD = D / 2, PITCH = D + 4;   // row pitch in floats: 16 consecutive rows start in different banks
  constexpr int DT = D / 32;                                     // dv tiles of the output accumulator
  constexpr int VPT = BKV * D / 4 / 256;                         // 16-byte vectors of a K (or V) tile per thread
  typedef __attribute__((ext_vector_type(4))) float f32x4s;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  float* smem = reinterpret_cast<float*>(smem_raw);              // [2 stages][K tile, V tile][BKV][PITCH]
  // Work items = (query tile, batch entry), the late (heavy, under the causal mask) query tiles first.  Several blocks
  // share a CU and the hardware deals consecutive block ids out CU after CU, so rounds of 256 block ids walk the item
  // list alternately forwards and backwards: the CU that got the heaviest item of one round gets the lightest of the next.
  unsigned item = blockIdx.x;
  if (a.heavyFirst == 2) item = ord.item[blockIdx.x];   // the host's table (see BlockOrder)
  else {
    const unsigned round = blockIdx.x >> 8, first = round << 8;
    const unsigned last = first + 255u < gridDim.x ? first + 255u : gridDim.x - 1u;
    if (round & 1u) item = last - (blockIdx.x - first);
  }
  const int qt = a.qTiles - 1 - (int)(item / (unsigned)a.nBatch);
  const LongType b = item % (unsigned)a.nBatch;
  if (a.H > 0) {
    const LongType hi = b / a.H, lo = b - hi * a.H;
    Q += hi * a.qB2 + lo * a.qB; K += hi * a.kB2 + lo * a.kB; V += hi * a.vB2 + lo * a.vB; O += hi * a.oB2 + lo * a.oB;
  } else {
    Q += b * a.qB; K += b * a.kB; V += b * a.vB; O += b * a.oB;
  }
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6, h = lane >> 5;
  const LongType q0 = (LongType)qt * BQ;
  const LongType query = q0 + wave * 32 + (lane & 31);
  const LongType qrow = query < a.Tq ? query : a.Tq - 1;
  const float L2E = 1.44269502162933349609375f;
  const float sc = a.applyScale ? a.scale : 1.f;

  float qf[HD];
#pragma unroll
  for (int i = 0; i < HD / 4; i++) {
    const f32x4s v = *reinterpret_cast<const f32x4s*>(Q + qrow * a.qT + h * HD + 4 * i);
    qf[4 * i] = v[0]; qf[4 * i + 1] = v[1]; qf[4 * i + 2] = v[2]; qf[4 * i + 3] = v[3];
  }
  f32x16 o[DT];
#pragma unroll
  for (int i = 0; i < DT; i++)
#pragma unroll
    for (int r = 0; r < 16; r++) o[i][r] = 0.f;
  float m = -1.0e30f, l = 0.f;

  LongType kvEnd = a.Tv;
  if (a.causal) { const LongType lim = q0 + BQ; kvEnd = lim < kvEnd ? lim : kvEnd; }
  const LongType nTiles = (kvEnd + BKV - 1) / BKV;

  // staging: vector i of this thread is (row, 16-byte column) = ((t + 256 i) / (D / 4), (t + 256 i) % (D / 4)) of the tile
  f32x4s kreg[VPT], vreg[VPT];
  auto fetch = [&](LongType kv0) {
#pragma unroll
    for (int i = 0; i < VPT; i++) {
      const int idx = t + 256 * i, row = idx / (D / 4), col = idx % (D / 4);
      LongType key = kv0 + row;
      key = key < a.Tv ? key : a.Tv - 1;              // keys past the end repeat the last one (their weights are exactly 0)
      kreg[i] = *reinterpret_cast<const f32x4s*>(K + key * a.kT + 4 * col);
      vreg[i] = *reinterpret_cast<const f32x4s*>(V + key * a.vT + 4 * col);
    }
  };
  auto park = [&](int stage) {
    float* sk = smem + stage * (2 * BKV * PITCH);
    float* sv = sk + BKV * PITCH;
#pragma unroll
    for (int i = 0; i < VPT; i++) {
      const int idx = t + 256 * i, row = idx / (D / 4), col = idx % (D / 4);
      *reinterpret_cast<f32x4s*>(sk + row * PITCH + 4 * col) = kreg[i];
      *reinterpret_cast<f32x4s*>(sv + row * PITCH + 4 * col) = vreg[i];
    }
  };
  if (nTiles > 0) { fetch(0); park(0); }
  __syncthreads();

  for (LongType it = 0; it < nTiles; it++) {
    const int cur = (int)(it & 1);
    const LongType kv0 = it * BKV;
    const float* sK = smem + cur * (2 * BKV * PITCH);
    const float* sV = sK + BKV * PITCH;
    const bool more = it + 1 < nTiles;
    if (more) fetch(kv0 + BKV);                       // in flight while this tile is multiplied

    // under the causal mask a wave sits out the tiles that lie wholly after its 32 queries (it still parks its share of
    // the next tile and meets the barrier)
    const bool idleWave = a.causal && kv0 > q0 + wave * 32 + 31;
    if (!idleWave) {
    // S^T = K Q^T for the 32 keys of the tile; two accumulators, so that consecutive MFMAs do not wait for each other
    f32x16 s, s2;
#pragma unroll
    for (int r = 0; r < 16; r++) { s[r] = 0.f; s2[r] = 0.f; }
    const float* krow = sK + (lane & 31) * PITCH + h * HD;
#pragma unroll
    for (int i = 0; i < HD / 4; i++) {
      const f32x4s kv = *reinterpret_cast<const f32x4s*>(krow + 4 * i);
      s = __builtin_amdgcn_mfma_f32_32x32x2f32(kv[0], qf[4 * i], s, 0, 0, 0);
      s2 = __builtin_amdgcn_mfma_f32_32x32x2f32(kv[1], qf[4 * i + 1], s2, 0, 0, 0);
      s = __builtin_amdgcn_mfma_f32_32x32x2f32(kv[2], qf[4 * i + 2], s, 0, 0, 0);
      s2 = __builtin_amdgcn_mfma_f32_32x32x2f32(kv[3], qf[4 * i + 3], s2, 0, 0, 0);
    }
#pragma unroll
    for (int r = 0; r < 16; r++) s[r] += s2[r];
    // register r: key kv0 + 8 (r / 4) + 4 h + r % 4 against this lane's query
    const bool edge = (a.causal && kv0 + BKV - 1 > q0 + wave * 32) || kv0 + BKV > a.Tv;
    float tmax = m;
#pragma unroll
    for (int r = 0; r < 16; r++) {
      float v = s[r] * sc;
      v = __builtin_fminf(__builtin_fmaxf(v, -1.0e4f), 1.0e4f);
      if (edge) {
        const LongType key = kv0 + 8 * (r >> 2) + 4 * h + (r & 3);
        if (key >= a.Tv || (a.causal && key > query)) v = -1.0e30f;
      }
      s[r] = v;
      tmax = __builtin_fmaxf(tmax, v);
    }
    tmax = __builtin_fmaxf(tmax, __shfl_xor(tmax, 32));
    const float alpha = __builtin_amdgcn_exp2f((m - tmax) * L2E);
    m = tmax;
    float psum = 0.f;
#pragma unroll
    for (int r = 0; r < 16; r++) {
      // a masked score (-1e30) sits 1e30 below the maximum whenever the row has seen a visible key; before that (m = -1e30
      // too) the difference is 0 and the weight must still be 0
      const float p = s[r] <= -1.0e30f ? 0.f : __builtin_amdgcn_exp2f((s[r] - m) * L2E);
      s[r] = p;
      psum += p;
    }
    psum += __shfl_xor(psum, 32);
    l = l * alpha + psum;
#pragma unroll
    for (int i = 0; i < DT; i++)
#pragma unroll
      for (int r = 0; r < 16; r++) o[i][r] *= alpha;
    // O^T += V^T P^T: step r pairs key 8 (r / 4) + 4 h + r % 4 of both half-waves
#pragma unroll
    for (int r = 0; r < 16; r++) {
      const float* vrow = sV + (8 * (r >> 2) + 4 * h + (r & 3)) * PITCH + (lane & 31);
#pragma unroll
      for (int i = 0; i < DT; i++) o[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(vrow[32 * i], s[r], o[i], 0, 0, 0);
    }
    }   // !idleWave
    if (more) park(cur ^ 1);                          // the other stage was last read before the barrier that ended the previous tile
    __syncthreads();
  }
  if (query < a.Tq) {
    const float inv = l > 0.f ? 1.f / l : 0.f;
    float* orow = O + query * a.oT;
#pragma unroll
    for (int i = 0; i < DT; i++)
#pragma unroll
      for (int g4 = 0; g4 < 4; g4++) {
        const f32x4s w = {o[i][4 * g4] * inv, o[i][4 * g4 + 1] * inv, o[i][4 * g4 + 2] * inv, o[i][4 * g4 + 3] * inv};
        *reinterpret_cast<f32x4s*>(orow + 32 * i + 8 * g4 + 4 * h) = w;
      }
  }
}
// The table of block order 2 for `nBatch` batch entries x `qTiles` query tiles under the causal mask, or null when the
// launch does not fit on the chip at once (`resident` blocks per CU) or in the table.  Items (heaviest query tile first)
// go one by one to the CU with the fewest key tiles so far that still has a block id left; with a multiple of 8 batch
// entries a batch entry stays on one XCD (block id mod 8), whose L2 then holds its K and V once.
static const BlockOrder* balancedBlockOrder(int nBatch, int qTiles, int keyTilesPerQueryTile, int resident) {
  const long total = (long)nBatch * qTiles;
  if (total > BLOCK_ORDER_MAX || total > 256L * resident || total <= 256 || qTiles < 2) return nullptr;
  static std::mutex mu;
  static std::map<std::array<int, 4>, std::unique_ptr<BlockOrder>> cache;
  std::lock_guard<std::mutex> lock(mu);
  auto& entry = cache[{nBatch, qTiles, keyTilesPerQueryTile, resident}];
  if (entry) return entry.get();
  for (int attempt = 0; attempt < 2; attempt++) {
    const bool byXcd = attempt == 0 && nBatch % 8 == 0;
    if (attempt == 0 && !byXcd) continue;
    auto t = std::make_unique<BlockOrder>();
    int cap[256], cnt[256] = {0};
    long load[256] = {0};
    for (int c = 0; c < 256; c++) cap[c] = c < total ? (int)((total - c + 255) / 256) : 0;
    bool ok = true;
    for (long p = 0; p < total && ok; p++) {
      const int slot = (int)(p / nBatch), b = (int)(p % nBatch);
      const long w = (long)keyTilesPerQueryTile * (qTiles - slot) + 1;   // key tiles of the query tile + the block's start-up
      int best = -1;
      for (int c = 0; c < 256; c++)
        if (cnt[c] < cap[c] && (!byXcd || (c & 7) == (b & 7)) && (best < 0 || load[c] < load[best])) best = c;
      if (best < 0) { ok = false; break; }
      t->item[cnt[best] * 256 + best] = (unsigned short)p;
      cnt[best]++; load[best] += w;
    }
    if (ok) { entry = std::move(t); return entry.get(); }
  }
  return nullptr;
}
static const BlockOrder& noBlockOrder() { static const BlockOrder z{}; return z; }
int attentionBlockOrder(int nBatch, int qTiles, int keyTilesPerQueryTile, int resident, unsigned short* items) {
  if (nBatch < 1 || qTiles < 1 || keyTilesPerQueryTile < 1 || resident < 1 || (long)nBatch * qTiles > BLOCK_ORDER_MAX) return 0;
  const BlockOrder* t = balancedBlockOrder(nBatch, qTiles, keyTilesPerQueryTile, resident);
  if (!t) return 0;
  for (int i = 0; i < nBatch * qTiles; i++) items[i] = t->item[i];
  return nBatch * qTiles;
}
// blocks of `kern` a CU holds at once
template <typename K>
static int residentBlocks(K kern, int ldsBytes) {
  int n = 0;
  if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, kern, 256, (size_t)ldsBytes) != hipSuccess) { (void)hipGetLastError(); return 0; }
  return n;
}

template <int D>
static void launchFusedF32(hipStream_t s, const void* q, const void* k, const void* v, void* out, const AttnDesc& d) {
  FusedArgs a;
  a.Tq = d.Tq; a.Tv = d.Tv;
  a.qB = d.qB; a.qT = d.qT; a.kB = d.kB; a.kT = d.kT; a.vB = d.vB; a.vT = d.vT; a.oB = d.oB; a.oT = d.oT;
  a.H = d.H; a.qB2 = d.qB2; a.kB2 = d.kB2; a.vB2 = d.vB2; a.oB2 = d.oB2;
  a.scale = d.scale; a.applyScale = d.applyScale ? 1 : 0; a.causal = d.causal ? 1 : 0;
  a.qTiles = (int)((d.Tq + 127) / 128); a.perBatch = a.qTiles; a.nBatch = (int)d.B; a.heavyFirst = 1;
  a.vmask = nullptr; a.maskValue = d.maskValue;
  constexpr int LDS = 2 * 2 * 32 * (D + 4) * 4;
  ND4J_REQUIRE((DynLds<attn_fused_f32<D>, LDS>::granted()), "attention: the device does not grant the fp32 fused kernel its LDS");
  static const int resident = residentBlocks(attn_fused_f32<D>, LDS);
  const BlockOrder* ord = d.causal && d.B * a.qTiles <= BLOCK_ORDER_MAX ? balancedBlockOrder((int)d.B, a.qTiles, 4, resident) : nullptr;
  if (ord) a.heavyFirst = 2;
  hipLaunchKernelGGL((attn_fused_f32<D>), dim3((unsigned)((LongType)a.qTiles * d.B)), dim3(256), LDS, s, a, ord ? *ord : noBlockOrder(), (const float*)q, (const float*)k,
                     (const float*)v, (float*)out);
}

bool attentionFusedSupported(DataType dt, const AttnDesc& d) {
  if (dt == FLOAT32) {
    if (d.vmask != nullptr || d.D != d.Dv || (d.D != 64 && d.D != 128) || d.Tq < 1 || d.Tv < 1) return false;
    for (LongType st : {d.qB, d.qT, d.kB, d.kT, d.vB, d.vT, d.oB, d.oT, d.qB2, d.kB2, d.vB2, d.oB2}) if (st % 4 != 0) return false;   // 16-byte aligned rows
    return ((d.Tq + 127) / 128) * d.B < (1LL << 31);
  }
  if (dt != HALF && dt != BFLOAT16) return false;
  if (d.D != d.Dv || (d.D != 64 && d.D != 128)) return false;
  if (d.Tq < 1 || d.Tv < 1) return false;
  // 16-byte aligned rows
  for (LongType st : {d.qB, d.qT, d.kB, d.kT, d.vB, d.vT, d.qB2, d.kB2, d.vB2}) if (st % 8 != 0) return false;
  if (d.oB % 4 != 0 || d.oT % 4 != 0 || d.oB2 % 4 != 0) return false;
  // the tile loads address a key inside a tile with a 32-bit byte offset
  if (d.kT < 0 || d.vT < 0 || d.kT >= (1 << 24) || d.vT >= (1 << 24)) return false;
  return true;
}

template <typename T, int D, bool FOLD, bool VM>
static void launchFusedTyped(hipStream_t s, const void* q, const void* k, const void* v, void* out, const AttnDesc& d) {
  FusedArgs a;
  a.Tq = d.Tq; a.Tv = d.Tv;
  a.qB = d.qB; a.qT = d.qT; a.kB = d.kB; a.kT = d.kT; a.vB = d.vB; a.vT = d.vT; a.oB = d.oB; a.oT = d.oT;
  a.H = d.H; a.qB2 = d.qB2; a.kB2 = d.kB2; a.vB2 = d.vB2; a.oB2 = d.oB2;
  a.scale = d.applyScale ? (float)d.scale : 1.f; a.applyScale = d.applyScale ? 1 : 0; a.causal = d.causal ? 1 : 0;
  a.qTiles = (int)((d.Tq + 127) / 128);
  a.nBatch = (int)d.B;
  a.vmask = d.vmask; a.maskValue = d.maskValue;
  a.perBatch = d.causal && !VM ? (a.qTiles + 1) / 2 : a.qTiles;   // with a value mask no key tile is skipped: equal tiles
  a.heavyFirst = 0;
  if (d.causal && !VM && a.qTiles > 1) {
    // time in key tiles per slot (a CU holds two blocks at D = 64, one at D = 128): equal paired blocks run in whole
    // rounds; single query tiles handed out heavy first finish within about a tenth of the mean, but not before the
    // longest tile.  The batch-major order keeps K and V closer, so it stays unless the rounds waste more than 8 %.
    const double slots = 256.0 * (D == 64 ? 2 : 1);
    const double pairCost = 2.0 * (a.qTiles + 1), pairs = (double)d.B * a.perBatch;
    const double pairedTime = std::ceil(pairs / slots) * pairCost;
    const double total = (double)d.B * a.qTiles * (a.qTiles + 1);
    const double heavyTime = std::max(1.1 * total / slots, 2.0 * a.qTiles);
    a.heavyFirst = pairedTime > 1.08 * heavyTime ? 1 : 0;
  }
  constexpr size_t LDS = (size_t)2 * ((D / 64) * 512 + 64 * (D / 8)) * 16;   // two stages of (K tile, V tile)
  auto kern = attn_fused<T, D, FOLD, VM>;
  ND4J_REQUIRE((DynLds<attn_fused<T, D, FOLD, VM>, (int)LDS>::granted()), "attention: the device does not grant the fused kernel its LDS");
  const BlockOrder* ord = nullptr;
  if (d.causal && !VM && a.qTiles > 1 && d.B * a.qTiles <= BLOCK_ORDER_MAX) {
    static const int resident = residentBlocks(kern, (int)LDS);
    ord = balancedBlockOrder((int)d.B, a.qTiles, 2, resident);
    if (ord) a.heavyFirst = 2;
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)((LongType)(a.heavyFirst ? a.qTiles : a.perBatch) * d.B)), dim3(256), LDS, s, a, ord ? *ord : noBlockOrder(), (const T*)q, (const T*)k,
                     (const T*)v, (T*)out);
}

void launchAttentionFused(hipStream_t s, DataType dt, const void* q, const void* k, const void* v, void* out, const AttnDesc& d) {
  ND4J_REQUIRE(attentionFusedSupported(dt, d), "attention: fused kernel does not take this problem");
  ND4J_REQUIRE((((uintptr_t)q | (uintptr_t)k | (uintptr_t)v) & 15) == 0 && ((uintptr_t)out & 7) == 0, "attention: operands must be 16-byte aligned");
  if (dt == FLOAT32) {
    ND4J_REQUIRE(((uintptr_t)out & 15) == 0, "attention: operands must be 16-byte aligned");
    if (d.D == 64) launchFusedF32<64>(s, q, k, v, out, d); else launchFusedF32<128>(s, q, k, v, out, d);
    HIP_CHECK(hipGetLastError());
    return;
  }
  ND4J_REQUIRE(((d.Tq + 127) / 128) * d.B < (1LL << 31), "attention: too many query tiles");
  // scale folded into the exponent: no scale at all, or bf16 scores with a power-of-two scale of moderate size (the
  // fp16 storage type has too narrow a range for rounding to commute with the scaling)
  const float sc = d.applyScale ? (float)d.scale : 1.f;
  int e = 0;
  const bool pow2 = sc > 0.f && std::frexp(sc, &e) == 0.5f && e >= -19 && e <= 21;
  const bool fold = sc == 1.f || (dt == BFLOAT16 && pow2);
  // the penalty of a masked logit is subtracted from the scaled logit, so the value-mask kernels keep the explicit scale
#define ND4J_FUSED(T, DD) (d.vmask ? launchFusedTyped<T, DD, false, true>(s, q, k, v, out, d) \
                           : fold ? launchFusedTyped<T, DD, true, false>(s, q, k, v, out, d) : launchFusedTyped<T, DD, false, false>(s, q, k, v, out, d))
  if (dt == HALF) { if (d.D == 64) ND4J_FUSED(f16_t, 64); else ND4J_FUSED(f16_t, 128); }
  else { if (d.D == 64) ND4J_FUSED(bf16_t, 64); else ND4J_FUSED(bf16_t, 128); }
#undef ND4J_FUSED
  HIP_CHECK(hipGetLastError());
}

}  // namespace nd4jhip
