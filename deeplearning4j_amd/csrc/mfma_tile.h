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

// Loader for one operand tile of `ROWS` rows (M or N index) x 64 k.
//   KC = true : memory is [row][k] with unit k stride; ld = row pitch
//   KC = false: memory is [k][row] with unit row stride; ld = k pitch
template <int ROWS, int NT, bool KC>
struct TileLoader {
  static constexpr int VECS = KC ? (ROWS * 8 + NT - 1) / NT : 0;        // 16-byte vectors per thread
  static constexpr int BLKS = KC ? 0 : (ROWS + NT - 1) / NT;            // 8x8 blocks per thread
  static constexpr int NREG = KC ? VECS : BLKS * 8;
  u32x4 reg[NREG > 0 ? NREG : 1];

  template <typename T>
  __device__ __forceinline__ void load(const T* __restrict__ base, LongType ld, LongType row0, LongType rowLimit, LongType k0, LongType K, int t) {
    const u32x4 zero = {0u, 0u, 0u, 0u};
    if (KC) {
#pragma unroll
      for (int i = 0; i < VECS; i++) {
        const int v = t + i * NT;
        if (VECS * NT != ROWS * 8 && v >= ROWS * 8) break;
        const int kg = v & 7, row = v >> 3;
        LongType r = row0 + row;
        r = r < rowLimit ? r : rowLimit - 1;
        const LongType k = k0 + kg * 8;
        reg[i] = k < K ? *reinterpret_cast<const u32x4*>(base + r * ld + k) : zero;
      }
    } else {
#pragma unroll
      for (int i = 0; i < BLKS; i++) {
        const int b = t + i * NT;
        if (BLKS * NT != ROWS && b >= ROWS) break;
        const int rb = b % (ROWS / 8), kg = b / (ROWS / 8);
        LongType r = row0 + rb * 8;
        r = r + 8 <= rowLimit ? r : rowLimit - 8;
#pragma unroll
        for (int q = 0; q < 8; q++) {
          const LongType k = k0 + kg * 8 + q;
          reg[i * 8 + q] = k < K ? *reinterpret_cast<const u32x4*>(base + k * ld + r) : zero;
        }
      }
    }
  }
  // lds: [8 k-groups][ROWS + 1] slots of 16 bytes
  __device__ __forceinline__ void store(u32x4* __restrict__ lds, LongType row0, LongType rowLimit, int t) {
    if (KC) {
#pragma unroll
      for (int i = 0; i < VECS; i++) {
        const int v = t + i * NT;
        if (VECS * NT != ROWS * 8 && v >= ROWS * 8) break;
        const int kg = v & 7, row = v >> 3;
        lds[kg * (ROWS + 1) + row] = reg[i];
      }
    } else {
#pragma unroll
      for (int i = 0; i < BLKS; i++) {
        const int b = t + i * NT;
        if (BLKS * NT != ROWS && b >= ROWS) break;
        const int rb = b % (ROWS / 8), kg = b / (ROWS / 8);
        u32x4 rows[8], cols[8];
#pragma unroll
        for (int q = 0; q < 8; q++) rows[q] = reg[i * 8 + q];
        transpose8x8(rows, cols);
        // a block clamped at the edge (row0 + rb*8 + 8 > rowLimit) was loaded from rowLimit-8: it is stored at
        // its nominal slot; its values belong to rows that the epilogue never writes
#pragma unroll
        for (int c = 0; c < 8; c++) lds[kg * (ROWS + 1) + rb * 8 + c] = cols[c];
      }
    }
  }
};

}  // namespace nd4jhip
