// Building blocks shared by the MFMA kernels (GEMM and fused attention): the 16-bit MFMA wrappers, the
// in-register 8x8 transpose and the operand tile loader that fills LDS in the [k/8][row][8 k-values] layout.
#pragma once
#include "device.h"

namespace nd4jhip {

typedef __attribute__((ext_vector_type(4))) unsigned u32x4;
typedef __attribute__((ext_vector_type(2))) unsigned u32x2;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;

template <typename T> struct Mfma16;
template <> struct Mfma16<f16_t> {
  static __device__ __forceinline__ f32x16 mma(u32x4 a, u32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
};
template <> struct Mfma16<bf16_t> {
  static __device__ __forceinline__ f32x16 mma(u32x4 a, u32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
};

// transpose an 8x8 block of 16-bit values held as 8 row vectors; out[c] collects element c of every row
__device__ __forceinline__ void transpose8x8(const u32x4 (&r)[8], u32x4 (&out)[8]) {
#pragma unroll
  for (int c = 0; c < 8; c++) {
    const unsigned sel = (c & 1) ? 0x07060302u : 0x05040100u;
#pragma unroll
    for (int d = 0; d < 4; d++) out[c][d] = __builtin_amdgcn_perm(r[2 * d + 1][c / 2], r[2 * d][c / 2], sel);
  }
}

// Loader for one operand tile of `ROWS` rows (M or N index) x 64 k, and the LDS layout it fills.
//   KC = true : memory is [row][k] with unit k stride; ld = row pitch.  16-byte vectors (8 k of one row) are
//               copied as they are.  LDS slot of (k-group kg, row r): kg * (ROWS + 1) + r.
//   KC = false: memory is [k][row] with unit row stride; ld = k pitch.  A thread loads a 4 (k) x 8 (rows) block,
//               transposes it in registers and writes eight 8-byte half-slots; neighbouring lanes hold the two
//               k-quads of one k-group, so a lane pair fills whole slots.  Rows are swizzled inside aligned groups
//               of 16, slot = kg * GROUP + (r ^ ((r >> 4) & 7)): the fragment reads (16 consecutive rows per
//               LDS pass) still cover 16 consecutive slots, and the writes of one instruction (fixed r % 8, lane
//               pairs = consecutive r / 8) land in 16 different slots modulo 16 -- both free of bank conflicts.
template <int ROWS, bool KC>
struct TileLayout {
  static constexpr int GROUP = KC ? ROWS + 1 : ROWS + 8;   // slots per k-group
  static constexpr int SLOTS = 8 * GROUP;                  // slots per 64-k tile
  static __device__ __forceinline__ int slot(int kg, int r) {
    return KC ? kg * GROUP + r : kg * GROUP + (r ^ ((r >> 4) & 7));
  }
};

// 16 bytes from an address that is only element-aligned (one global_load_dwordx4: the platform runs global memory in
// unaligned access mode and the compiler emits the wide load itself for such a copy)
__device__ __forceinline__ u32x4 load16u(const void* p) {
  u32x4 v;
  __builtin_memcpy(&v, p, 16);
  return v;
}
// the same through a non-temporal load: for operands that are read once and are large against the last-level cache
// (a vocabulary's embedding under a few rows of activations), so that they do not push out what is read again
template <bool NT>
__device__ __forceinline__ u32x4 load16u_stream(const void* p) {
  if constexpr (NT) {
    typedef unsigned u32x4_elem __attribute__((ext_vector_type(4), aligned(2)));
    return __builtin_bit_cast(u32x4, __builtin_nontemporal_load(reinterpret_cast<const u32x4_elem*>(p)));
  } else {
    return load16u(p);
  }
}
// the eight 16-bit elements of v moved down by sh places: element j + sh lands in place j, zeros come in from the top
// (sh >= 8: all zeros).  Selects only, no indexed register access.
__device__ __forceinline__ u32x4 shiftDownElems(u32x4 v, int sh) {
  const int ds = sh >> 1;
  const bool odd = (sh & 1) != 0;
  auto pick = [&](int idx) -> unsigned { return idx == 0 ? v[0] : idx == 1 ? v[1] : idx == 2 ? v[2] : idx == 3 ? v[3] : 0u; };
  u32x4 o;
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const unsigned lo = pick(ds + i), hi = pick(ds + i + 1);
    o[i] = odd ? (lo >> 16) | (hi << 16) : lo;
  }
  return o;
}

template <int ROWS, int NT, bool KC>
struct TileLoader {
  using Layout = TileLayout<ROWS, KC>;
  static constexpr int UNITS = KC ? ROWS * 8 : ROWS * 2;                 // vectors / 4x8 blocks per tile
  static constexpr int PER = (UNITS + NT - 1) / NT;                      // per thread
  static constexpr int NREG = KC ? PER : PER * 4;
  u32x4 reg[NREG];

  // The loader of the kernels that handle ragged shapes.  Rows need element alignment only (any row pitch, any start), and the
  // contiguous extent need not be a multiple of 8: every load is an unconditional 16-byte read from a position inside the
  // operand -- a group that would run over the end of its row (k-contiguous operand: k + 8 > K; row-contiguous operand: the
  // last rows) is read 8 elements back from the end instead and moved down in registers, zeros coming in for what lies
  // beyond; k positions past K give zeros (they meet the other operand's tail); rows past the limit of a k-contiguous
  // operand repeat the last row (their products are never stored).  Needs K >= 8 (k-contiguous) or rowLimit >= 8.
  template <typename T, bool STREAM = false>
  __device__ __forceinline__ void load(const T* __restrict__ base, LongType ld, LongType row0, LongType rowLimit, LongType k0, LongType K, int t) {
    const u32x4 zero = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int i = 0; i < PER; i++) {
      const int u = t + i * NT;
      if (PER * NT != UNITS && u >= UNITS) break;
      if (KC) {
        const int kg = u & 7, row = u >> 3;
        LongType r = row0 + row;
        r = r < rowLimit ? r : rowLimit - 1;
        const LongType k = k0 + kg * 8;
        const LongType kk = k + 8 <= K ? k : K - 8;
        reg[i] = load16u_stream<STREAM>(base + r * ld + kk);
        if (k != kk) reg[i] = shiftDownElems(reg[i], (int)(k - kk < 8 ? k - kk : 8));
      } else {
        const int rb = (u >> 1) % (ROWS / 8), kq = (u / (ROWS / 4)) * 2 + (u & 1);   // 8-row block, 4-k quad (16 per tile)
        const LongType r = row0 + rb * 8;
        const LongType rr = r + 8 <= rowLimit ? r : rowLimit - 8;
        const int sh = (int)(r - rr < 8 ? r - rr : 8);
#pragma unroll
        for (int q = 0; q < 4; q++) {
          const LongType k = k0 + kq * 4 + q;
          reg[i * 4 + q] = load16u_stream<STREAM>(base + (k < K ? k : K - 1) * ld + rr);
        }
#pragma unroll
        for (int q = 0; q < 4; q++) {
          if (k0 + kq * 4 + q >= K) reg[i * 4 + q] = zero;
          else if (sh) reg[i * 4 + q] = shiftDownElems(reg[i * 4 + q], sh);
        }
      }
    }
  }
  // load() without predicates: rows and k positions past the end are clamped to the last valid one instead of being
  // zero-filled (the caller never uses what they hold, but it must be finite data).  Every load is unconditional, so
  // the compiler places its wait where the registers are consumed instead of at the join after each predicated load.
  // Needs K - k0 to be a multiple of 8 for a k-contiguous operand (whole 16-byte k-groups).
  template <typename T>
  __device__ __forceinline__ void loadClamped(const T* __restrict__ base, LongType ld, LongType row0, LongType rowLimit, LongType k0, LongType K, int t) {
#pragma unroll
    for (int i = 0; i < PER; i++) {
      const int u = t + i * NT;
      if (PER * NT != UNITS && u >= UNITS) break;
      if (KC) {
        const int kg = u & 7, row = u >> 3;
        LongType r = row0 + row;
        r = r < rowLimit ? r : rowLimit - 1;
        LongType k = k0 + kg * 8;
        k = k < K ? k : K - 8;
        reg[i] = *reinterpret_cast<const u32x4*>(base + r * ld + k);
      } else {
        const int rb = (u >> 1) % (ROWS / 8), kq = (u / (ROWS / 4)) * 2 + (u & 1);
        LongType r = row0 + rb * 8;
        r = r + 8 <= rowLimit ? r : rowLimit - 8;
#pragma unroll
        for (int q = 0; q < 4; q++) {
          LongType k = k0 + kq * 4 + q;
          k = k < K ? k : K - 1;
          reg[i * 4 + q] = *reinterpret_cast<const u32x4*>(base + k * ld + r);
        }
      }
    }
  }
  // same as load() for a tile that lies wholly inside the operand: no clamping, no predicates
  template <typename T>
  __device__ __forceinline__ void loadFull(const T* __restrict__ base, LongType ld, LongType row0, LongType k0, int t) {
#pragma unroll
    for (int i = 0; i < PER; i++) {
      const int u = t + i * NT;
      if (PER * NT != UNITS && u >= UNITS) break;
      if (KC) {
        reg[i] = *reinterpret_cast<const u32x4*>(base + (row0 + (u >> 3)) * ld + k0 + (u & 7) * 8);
      } else {
        const int rb = (u >> 1) % (ROWS / 8), kq = (u / (ROWS / 4)) * 2 + (u & 1);
#pragma unroll
        for (int q = 0; q < 4; q++) reg[i * 4 + q] = *reinterpret_cast<const u32x4*>(base + (k0 + kq * 4 + q) * ld + row0 + rb * 8);
      }
    }
  }
  __device__ __forceinline__ void store(u32x4* __restrict__ lds, int t) {
#pragma unroll
    for (int i = 0; i < PER; i++) {
      const int u = t + i * NT;
      if (PER * NT != UNITS && u >= UNITS) break;
      if (KC) {
        lds[Layout::slot(u & 7, u >> 3)] = reg[i];
      } else {
        const int rb = (u >> 1) % (ROWS / 8), kq = (u / (ROWS / 4)) * 2 + (u & 1);
        // column c of the 4x8 block: k = kq*4 .. +3 of row rb*8 + c -> half (kq & 1) of slot (kq / 2, row).
        // A block clamped at the tile edge holds values of rows that the epilogue never writes.
#pragma unroll
        for (int c = 0; c < 8; c++) {
          const unsigned sel = (c & 1) ? 0x07060302u : 0x05040100u;
          u32x2 w;
          w[0] = __builtin_amdgcn_perm(reg[i * 4 + 1][c / 2], reg[i * 4 + 0][c / 2], sel);
          w[1] = __builtin_amdgcn_perm(reg[i * 4 + 3][c / 2], reg[i * 4 + 2][c / 2], sel);
          reinterpret_cast<u32x2*>(&lds[Layout::slot(kq >> 1, rb * 8 + c)])[kq & 1] = w;
        }
      }
    }
  }
};

// Loader for a 64 (k) x ROWS tile of an operand stored [k][row] with unit row stride, kept in LDS as it lies in memory
// (no register transpose): the fragments are taken with the transposing LDS read (ds_read_b64_tr_b16), which hands a lane
// the four k-values of one row out of a 4 (k) x 16 (rows) block read by its 16-lane group.  A k-row is ROWS / 8 slots of
// 16 bytes; slot s of k-row k sits at k * (ROWS / 8) + (s ^ swz(k)).  The swizzle keeps the read free of bank
// conflicts: 32 lanes fetch 4 k-rows x 64 bytes per pass, and k-rows whose starts fall on the same bank (every second
// one for 128-byte rows, all of them from 256-byte rows on) are moved to different 64-byte quarters of the row.
template <int ROWS, int NT>
struct RowTileLoader {
  static_assert(ROWS >= 64 && ROWS % 64 == 0, "a k-row holds whole 128-byte lines");
  static constexpr int SPR = ROWS / 8;              // slots per k-row
  static constexpr int UNITS = 64 * SPR, PER = (UNITS + NT - 1) / NT;
  static_assert(UNITS % NT == 0, "every thread moves the same number of vectors");
  u32x4 reg[PER];
  static __device__ __forceinline__ int swz(int k) { return ROWS == 64 ? 4 * ((k >> 1) & 1) : 4 * (k & 3); }
  template <typename T>
  __device__ __forceinline__ void loadFull(const T* __restrict__ base, LongType ld, LongType row0, LongType k0, int t) {
#pragma unroll
    for (int i = 0; i < PER; i++) {
      const int u = t + i * NT;
      reg[i] = *reinterpret_cast<const u32x4*>(base + (k0 + u / SPR) * ld + row0 + (u % SPR) * 8);
    }
  }
  __device__ __forceinline__ void store(u32x4* __restrict__ lds, int t) {
#pragma unroll
    for (int i = 0; i < PER; i++) {
      const int u = t + i * NT, k = u / SPR;
      lds[k * SPR + ((u % SPR) ^ swz(k))] = reg[i];
    }
  }
  // Byte offset (inside the tile) of the lane's first transposing read for the 32 rows starting at row32 and k-step 0;
  // k-step ks adds ks * 16 k-rows, the second read of a k-step (k-values 4..7 of the lane's eight) adds 4 k-rows.
  static __device__ __forceinline__ int fragOffset(int row32, int lane) {
    const int grp = lane >> 4, i16 = lane & 15;
    const int r4 = row32 + 16 * (grp & 1) + 4 * (i16 & 3);
    const int k = 8 * (grp >> 1) + (i16 >> 2);
    return (k * SPR + ((r4 >> 3) ^ swz(k))) * 16 + ((r4 >> 2) & 1) * 8;
  }
  static constexpr int KSTEP_BYTES = 16 * SPR * 16, HALF_BYTES = 4 * SPR * 16;
  static __device__ __forceinline__ u32x4 readFrag(const u32x4* tile, int fragOff, int ks) {
    typedef __attribute__((address_space(3))) void* lds_ptr;
    typedef short s16x4 __attribute__((ext_vector_type(4)));
    const __attribute__((address_space(3))) unsigned char* base =
        (const __attribute__((address_space(3))) unsigned char*)(lds_ptr)tile + fragOff + ks * KSTEP_BYTES;
    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)base);
    const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(base + HALF_BYTES));
    const u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
    return u32x4{l2[0], l2[1], h2[0], h2[1]};
  }
};

}  // namespace nd4jhip
