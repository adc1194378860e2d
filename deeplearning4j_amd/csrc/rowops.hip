// Row kernels: softmax and layer_norm.
//
// softmax (reference: libnd4j/include/ops/declarable/helpers/cpu/softmax.cpp:252-353)
//   One wave (rows up to 64*NV*VEC elements) or one 256-thread block owns a row and keeps it in
//   registers: one read of x, one write of z => algorithmic bytes 2*sizeof(T) per element, HBM-bound.
//   Rows sit at offsets given by the outer dims of input and output separately, so a permuted input
//   view with a contiguous last axis runs at the same speed as a dense one.
//   clamp mode reproduces the reference's same-shape branch: max over finite values (0 if none),
//   inf/nan mapped to max+-88, diff clamped to +-88, sum floored at 1e-6.  Plain mode is the fallback
//   branch (max, sub, exp, sum, div).  All arithmetic in float (double for fp64 arrays).
//
// layer_norm (reference: generic/nn/layer_norm.cpp:35-79 = standardize (generic/transforms/
//   standardize.cpp:34-78) * gain + bias): one fused pass instead of the reference's eight:
//   mean, population variance, y = (x - mean) / sqrt(var + 1e-5) * gain + bias.
#include "device.h"
#include "rowmath.h"
#include "kernels.h"
#include "runtime.h"

namespace nd4jhip {

struct RowArgs {
  DevShape outerX, outerZ;
  LongType rows, rowLen, xInner, zInner;
};

template <typename A> __device__ __forceinline__ A r_exp(A x);
template <> __device__ __forceinline__ float r_exp<float>(float x) { return expf(x); }
template <> __device__ __forceinline__ double r_exp<double>(double x) { return exp(x); }
template <typename A> __device__ __forceinline__ bool r_finite(A x) { return x == x && x != (A)INFINITY && x != -(A)INFINITY; }
template <typename A> __device__ __forceinline__ A r_tmax();
template <> __device__ __forceinline__ float r_tmax<float>() { return 3.4028234663852886e38f; }
template <> __device__ __forceinline__ double r_tmax<double>() { return 1.7976931348623157e308; }

template <typename Op, int TPR, typename A>
__device__ __forceinline__ A row_allreduce(A v, A* lds) {
  if (TPR == 64) return wave_allreduce<Op>(v);
  return block_allreduce<Op, 4, A>(v, lds);
}

// softmax numerator of one value given the row max.  Clamp mode: finite x gives exp(max(x - max, -88)) (the
// upper clamp can only bind for +inf/NaN, which the reference maps to max + 88); plain mode: exp(x - max).
// The exponential is v_exp_f32 on d*log2(e): its error relative to the row's largest term is below 3e-8.
__device__ __forceinline__ float softmax_term(float v, float mx, int clamp) {
  const float L2E = 1.44269502162933349609375f;
  float d = v - mx;
  if (clamp) {
    d = __builtin_fmaxf(d, -88.f);                      // -inf and finite underflow; a NaN operand is dropped
    d = (v <= 3.4028234663852886e38f) ? d : 88.f;       // +inf and NaN take the upper clamp
  }
  return __builtin_amdgcn_exp2f(d * L2E);
}
__device__ __forceinline__ double softmax_term(double v, double mx, int clamp) {
  if (clamp) {
    if (!r_finite(v)) v = (v > 0 || v != v) ? 88.0 + mx : -88.0 + mx;
    double d = v - mx;
    d = d > 88.0 ? 88.0 : d;
    d = d < -88.0 ? -88.0 : d;
    return exp(d);
  }
  return exp(v - mx);
}
// max over the finite values only (clamp mode) folded into one compare + select
template <typename A>
__device__ __forceinline__ A softmax_maxstep(A mx, A v, int clamp) {
  if (clamp) v = (v < 0 ? -v : v) <= r_tmax<A>() ? v : -r_tmax<A>();
  return v > mx ? v : mx;
}

// VEC == 1: element loads through xInner/zInner strides; VEC > 1: 16-byte loads, unit strides
template <typename T, int TPR, int NV, int VEC>
__global__ __launch_bounds__(256) void softmax_rows(RowArgs a, const T* __restrict__ x, T* __restrict__ z, int clamp, int nt) {
  using A = typename Conv<T>::acc;
  using VT = Vec<T, VEC>;
  constexpr int ROWS = 256 / TPR;
  __shared__ A lds[4];
  const int t = threadIdx.x % TPR;
  LongType row = (LongType)blockIdx.x * ROWS + threadIdx.x / TPR;
  const bool live = row < a.rows;
  if (!live) row = a.rows - 1;  // keep the wave convergent for the block-wide reductions
  const LongType xb = walk<LongType>(a.outerX, row), zb = walk<LongType>(a.outerZ, row);
  const LongType L = a.rowLen;
  A vals[NV * VEC];
  const A NEG = -r_tmax<A>();
#pragma unroll
  for (int i = 0; i < NV; i++) {
    const LongType e0 = ((LongType)t + (LongType)i * TPR) * VEC;
    if (VEC > 1) {
      if (e0 < L) {
        const typename RawIO<T>::raw* src = reinterpret_cast<const typename RawIO<T>::raw*>(x + xb + e0);
        RawIO<T>::unpack(nt == 1 ? __builtin_nontemporal_load(src) : *src, &vals[i * VEC]);
      } else {
#pragma unroll
        for (int e = 0; e < VEC; e++) vals[i * VEC + e] = NEG;
      }
    } else {
      vals[i] = e0 < L ? (A)to_float(x[xb + e0 * a.xInner]) : NEG;
    }
  }
  A mx = NEG, sum = (A)0;
  // Rows of finite numbers (all of them, in practice) need neither the finite-only maximum nor the +-88 clamps:
  // below -88 the clamp would put e^-88 = 6e-39 where this path puts a smaller number or 0, far below what the
  // output type or the sum can resolve.  0 * v is NaN exactly for v = +-inf or NaN, which makes a one-instruction
  // probe; padding slots hold -FLT_MAX and contribute exp2(-inf) = 0 without a bounds test.
  bool fast = false;
  if (TPR == 64 && sizeof(A) == 4) {
    A probe = (A)0;
#pragma unroll
    for (int i = 0; i < NV * VEC; i++) {
      probe = __builtin_fmaf((float)vals[i], 0.f, (float)probe);
      mx = vals[i] > mx ? vals[i] : mx;
    }
    fast = __builtin_amdgcn_ballot_w64(probe != probe) == 0;
  }
  if (fast) {
    mx = row_allreduce<MaxOp, TPR, A>(mx, lds);
    const float L2E = 1.44269502162933349609375f;
#pragma unroll
    for (int i = 0; i < NV * VEC; i++) {
      const A r = (A)__builtin_amdgcn_exp2f(((float)vals[i] - (float)mx) * L2E);
      vals[i] = r;
      sum += r;
    }
  } else {
    mx = NEG;
#pragma unroll
    for (int i = 0; i < NV * VEC; i++) {
      mx = softmax_maxstep<A>(mx, vals[i], clamp);
    }
    mx = row_allreduce<MaxOp, TPR, A>(mx, lds);
    if (clamp && mx == NEG) mx = (A)0;
#pragma unroll
    for (int i = 0; i < NV; i++) {
      const LongType e0 = ((LongType)t + (LongType)i * TPR) * VEC;
#pragma unroll
      for (int e = 0; e < VEC; e++) {
        if (e0 + e < L) { A r = softmax_term(vals[i * VEC + e], mx, clamp); vals[i * VEC + e] = r; sum += r; }
      }
    }
  }
  sum = row_allreduce<SumOp, TPR, A>(sum, lds);
  if (clamp) sum = sum > (A)1e-6f ? sum : (A)1e-6f;
  if (!live) return;
  const A inv = (A)1 / sum;   // one division per row; every element is scaled by the reciprocal
#pragma unroll
  for (int i = 0; i < NV; i++) {
    const LongType e0 = ((LongType)t + (LongType)i * TPR) * VEC;
    if (e0 >= L) continue;
    if (VEC > 1) {
#pragma unroll
      for (int e = 0; e < VEC; e++) vals[i * VEC + e] *= inv;
      typename RawIO<T>::raw* dst = reinterpret_cast<typename RawIO<T>::raw*>(z + zb + e0);
      store_vec(dst, RawIO<T>::pack(&vals[i * VEC]), nt != 0);
    } else {
      z[zb + e0 * a.zInner] = Conv<T>::from(vals[i] * inv);
    }
  }
}

// Rows with unit inner stride that fit one wave's registers (softmax over the contiguous last axis of a dense array or of a
// permuted view): every load unconditional (lanes past the row's end re-read its last vector and their bits are replaced
// by the padding value) and pinned ahead of the first use, one wave per row.
// Measured on fp32 [196608, 1024]: 253 us against 275 us for the general kernel (a plain copy of the same bytes: 242 us).
template <typename T> struct PadBits;   // the 16-bit / 32-bit pattern of -max(T), repeated over a 32-bit word
template <> struct PadBits<float> { static constexpr unsigned v = 0xff7fffffu; };
template <> struct PadBits<bf16_t> { static constexpr unsigned v = 0xff7fff7fu; };
template <> struct PadBits<f16_t> { static constexpr unsigned v = 0xfbfffbffu; };
// G: lanes per row (64: a wave per row; 8, 16, 32: several short rows per wave, NV == 1)
// NT: 1 = non-temporal loads and stores (arrays beyond the last-level cache), 2 = stores only (results of 8 MiB and more)
template <typename T, int NV, int NT, int G = 64>
__global__ __launch_bounds__(256) void softmax_linear(RowArgs a, const T* __restrict__ x, T* __restrict__ z, int clamp) {
  using Raw = typename RawIO<T>::raw;
  constexpr int VEC = RawIO<T>::N;
  const int t = threadIdx.x & (G - 1);
  const LongType row = (LongType)blockIdx.x * (256 / G) + threadIdx.x / G;
  if (row >= a.rows) return;
  const int L = (int)a.rowLen;
  const T* xr = x + walk<LongType>(a.outerX, row);
  raw_u32x4 bits[NV];
  int e0[NV];
#pragma unroll
  for (int i = 0; i < NV; i++) {
    const int e = (t + i * G) * VEC;
    e0[i] = e < L ? e : L - VEC;
    const raw_u32x4* src = reinterpret_cast<const raw_u32x4*>(xr + e0[i]);
    bits[i] = NT == 1 ? __builtin_nontemporal_load(src) : *src;
  }
  __builtin_amdgcn_sched_barrier(0);   // all loads are issued before the first use: one trip to memory per row
  float vals[NV * VEC];
  const float NEG = -r_tmax<float>();
#pragma unroll
  for (int i = 0; i < NV; i++) {
    const unsigned keep = (t + i * G) * VEC < L ? 0xffffffffu : 0u;
    const raw_u32x4 b = (bits[i] & keep) | (raw_u32x4)(PadBits<T>::v & ~keep);
    RawIO<T>::unpack(__builtin_bit_cast(Raw, b), &vals[i * VEC]);
  }
  // rows of finite numbers need neither the finite-only maximum nor the +-88 clamps (see softmax_rows); 0 * v is NaN
  // exactly for v = +-inf or NaN; the padding (-max) is finite
  float mx = NEG, probe = 0.f;
#pragma unroll
  for (int i = 0; i < NV * VEC; i++) {
    probe = __builtin_fmaf(vals[i], 0.f, probe);
    mx = vals[i] > mx ? vals[i] : mx;
  }
  float sum = 0.f;
  const float L2E = 1.44269502162933349609375f;
  if (__builtin_amdgcn_ballot_w64(probe != probe) == 0) {
    mx = group_allreduce<MaxOp, G>(mx);
#pragma unroll
    for (int i = 0; i < NV * VEC; i++) {
      const float r = __builtin_amdgcn_exp2f((vals[i] - mx) * L2E);
      vals[i] = r;
      sum += r;
    }
  } else {
    mx = NEG;
#pragma unroll
    for (int i = 0; i < NV * VEC; i++) mx = softmax_maxstep<float>(mx, vals[i], clamp);
    mx = group_allreduce<MaxOp, G>(mx);
    if (clamp && mx == NEG) mx = 0.f;
#pragma unroll
    for (int i = 0; i < NV; i++)
#pragma unroll
      for (int e = 0; e < VEC; e++) {
        float r = 0.f;
        if ((t + i * G) * VEC < L) r = softmax_term(vals[i * VEC + e], mx, clamp);
        vals[i * VEC + e] = r;
        sum += r;
      }
  }
  sum = group_allreduce<SumOp, G>(sum);
  if (clamp) sum = sum > 1e-6f ? sum : 1e-6f;
  const float inv = 1.f / sum;
  T* zr = z + walk<LongType>(a.outerZ, row);
#pragma unroll
  for (int i = 0; i < NV; i++) {
    if ((t + i * G) * VEC >= L) continue;
#pragma unroll
    for (int e = 0; e < VEC; e++) vals[i * VEC + e] *= inv;
    Raw* dst = reinterpret_cast<Raw*>(zr + e0[i]);
    if (NT) __builtin_nontemporal_store(RawIO<T>::pack(&vals[i * VEC]), dst);
    else *dst = RawIO<T>::pack(&vals[i * VEC]);
  }
}

// rows longer than the register budget: three passes over global memory, one block per row
template <typename T>
__global__ __launch_bounds__(256) void softmax_long(RowArgs a, const T* __restrict__ x, T* __restrict__ z, int clamp) {
  using A = typename Conv<T>::acc;
  __shared__ A lds[4];
  const LongType row = blockIdx.x;
  const LongType xb = walk<LongType>(a.outerX, row), zb = walk<LongType>(a.outerZ, row);
  const A NEG = -r_tmax<A>();
  A mx = NEG;
  for (LongType j = threadIdx.x; j < a.rowLen; j += 256) {
    mx = softmax_maxstep<A>(mx, (A)to_float(x[xb + j * a.xInner]), clamp);
  }
  mx = block_allreduce<MaxOp, 4, A>(mx, lds);
  if (clamp && mx == NEG) mx = (A)0;
  A sum = (A)0;
  for (LongType j = threadIdx.x; j < a.rowLen; j += 256) sum += softmax_term((A)to_float(x[xb + j * a.xInner]), mx, clamp);
  sum = block_allreduce<SumOp, 4, A>(sum, lds);
  if (clamp) sum = sum > (A)1e-6f ? sum : (A)1e-6f;
  for (LongType j = threadIdx.x; j < a.rowLen; j += 256)
    z[zb + j * a.zInner] = Conv<T>::from(softmax_term((A)to_float(x[xb + j * a.xInner]), mx, clamp) / sum);
}

template <typename A> __device__ __forceinline__ A r_log(A x);
template <> __device__ __forceinline__ float r_log<float>(float x) { return logf(x); }
template <> __device__ __forceinline__ double r_log<double>(double x) { return log(x); }
// The same for unit-stride rows (a vocabulary's worth of logits): one block of 1024 threads per row, 16-byte loads four at a
// time per thread.  A row may start anywhere (rows of an odd length do): the elements up to the first 16-byte boundary and
// after the last whole vector are read one by one; x and z must sit at the same offset from such a boundary.  The row is read
// from memory once and twice more from the cache it fits in; the exponential is taken twice per element, as above.
template <typename T, bool LOG = false>
__global__ __launch_bounds__(1024) void softmax_long_vec(RowArgs a, const T* __restrict__ x, T* __restrict__ z, int clamp) {
  using A = typename Conv<T>::acc;
  using Raw = typename RawIO<T>::raw;
  constexpr int VEC = RawIO<T>::N, NT = 1024, UNR = 4;
  __shared__ A lds[NT / 64];
  const LongType row = blockIdx.x;
  const T* xr = x + walk<LongType>(a.outerX, row);
  T* zr = z + walk<LongType>(a.outerZ, row);
  const LongType L = a.rowLen;
  const int t = threadIdx.x;
  LongType head = (LongType)(((16 - (reinterpret_cast<uintptr_t>(xr) & 15)) & 15) / sizeof(T));
  if (head > L) head = L;
  const LongType nv = (L - head) / VEC, tail0 = head + nv * VEC;
  const Raw* xv = reinterpret_cast<const Raw*>(xr + head);
  // f(value, position) over the whole row: head and tail element by element, the body UNR vectors per thread and trip
  auto sweep = [&](auto&& f) {
    for (LongType j = t; j < head; j += NT) f((A)to_float(xr[j]), j);
    for (LongType j = tail0 + t; j < L; j += NT) f((A)to_float(xr[j]), j);
    for (LongType i = t; i < nv; i += (LongType)UNR * NT) {
      Raw v[UNR];
#pragma unroll
      for (int u = 0; u < UNR; u++) { const LongType iu = i + (LongType)u * NT; v[u] = xv[iu < nv ? iu : nv - 1]; }
#pragma unroll
      for (int u = 0; u < UNR; u++) {
        const LongType iu = i + (LongType)u * NT;
        if (iu < nv) {
          A vals[VEC];
          RawIO<T>::unpack(v[u], vals);
#pragma unroll
          for (int e = 0; e < VEC; e++) f(vals[e], head + iu * VEC + e);
        }
      }
    }
  };
  const A NEG = -r_tmax<A>();
  A mx = NEG;
  sweep([&](A v, LongType) { mx = LOG ? (v > mx ? v : mx) : softmax_maxstep<A>(mx, v, clamp); });
  if constexpr (NT == 64) mx = wave_allreduce<MaxOp>(mx); else mx = block_allreduce<MaxOp, NT / 64, A>(mx, lds);
  if (!LOG && clamp && mx == NEG) mx = (A)0;
  A sum = (A)0;
  // LOG: log(exp(x - max) / sum) in that order, as log_softmax_rows evaluates it
  auto term = [&](A v) -> A { if constexpr (LOG) return r_exp<A>(v - mx); else return softmax_term(v, mx, clamp); };
  sweep([&](A v, LongType) { sum += term(v); });
  sum = block_allreduce<SumOp, NT / 64, A>(sum, lds);
  if (!LOG && clamp) sum = sum > (A)1e-6f ? sum : (A)1e-6f;
  auto result = [&](A v) -> A { if constexpr (LOG) return r_log<A>(term(v) / sum); else return term(v) / sum; };
  // the result: whole vectors where whole vectors were read
  for (LongType j = t; j < head; j += NT) zr[j] = Conv<T>::from(result((A)to_float(xr[j])));
  for (LongType j = tail0 + t; j < L; j += NT) zr[j] = Conv<T>::from(result((A)to_float(xr[j])));
  Raw* zv = reinterpret_cast<Raw*>(zr + head);
  for (LongType i = t; i < nv; i += (LongType)UNR * NT) {
    Raw v[UNR];
#pragma unroll
    for (int u = 0; u < UNR; u++) { const LongType iu = i + (LongType)u * NT; v[u] = xv[iu < nv ? iu : nv - 1]; }
#pragma unroll
    for (int u = 0; u < UNR; u++) {
      const LongType iu = i + (LongType)u * NT;
      if (iu < nv) {
        A vals[VEC];
        RawIO<T>::unpack(v[u], vals);
#pragma unroll
        for (int e = 0; e < VEC; e++) vals[e] = result(vals[e]);
        zv[iu] = RawIO<T>::pack(vals);
      }
    }
  }
}

// Unit-stride rows of up to NV x 512 vectors (fp32 up to 65,536 values, 16-bit up to 131,072: a vocabulary's logits): one
// block of 512 threads (two waves per SIMD: 256 registers each) holds the whole row in registers, so it comes from memory once and the three passes (maximum, sum of
// exponentials, result) run on registers.  Rows may start anywhere: the 16-byte loads and stores are element-aligned (global
// memory runs in unaligned access mode), the values after the last whole vector go one per thread.
// NT = 64: a wave per row, four rows to a block of 256 threads -- rows of up to NV x 64 vectors whose starts or length keep
// them off the aligned vector kernels (attention scores of a 1001-token prompt: bf16 [192, 1001, 1001] 2.4 -> see the launcher).
template <typename T, int NV, bool LOG, bool NTS = false, int NT = 512>
__global__ __launch_bounds__(NT == 64 ? 256 : NT) void softmax_block_regs(RowArgs a, const T* __restrict__ x, T* __restrict__ z, int clamp) {
  using A = typename Conv<T>::acc;
  using Raw = typename RawIO<T>::raw;
  constexpr int VEC = RawIO<T>::N;
  static_assert(NT == 512 || NT == 64, "a block of 512 threads or a wave per row");
  __shared__ A lds[NT == 64 ? 1 : NT / 64];
  const LongType row = NT == 64 ? (LongType)blockIdx.x * 4 + threadIdx.x / 64 : (LongType)blockIdx.x;
  if (NT == 64 && row >= a.rows) return;
  const T* xr = x + walk<LongType>(a.outerX, row);
  T* zr = z + walk<LongType>(a.outerZ, row);
  const LongType L = a.rowLen, nv = L / VEC, tail0 = nv * VEC;
  const int t = NT == 64 ? (int)(threadIdx.x & 63) : (int)threadIdx.x;
  Raw v[NV];
#pragma unroll
  for (int i = 0; i < NV; i++) {
    const LongType iv = (LongType)i * NT + t;
    __builtin_memcpy(&v[i], xr + (iv < nv ? iv : nv - 1) * VEC, sizeof(Raw));
  }
  const bool hasTail = tail0 + t < L;
  const A tailv = hasTail ? (A)to_float(xr[tail0 + t]) : (A)0;
  auto sweep = [&](auto&& f) {
#pragma unroll
    for (int i = 0; i < NV; i++) {
      if ((LongType)i * NT + t < nv) {
        A vals[VEC];
        // (16-bit rows: the opaque pass keeps the compiler from holding the unpacked row, twice or four times the registers)
        if constexpr (sizeof(T) == 2 && NV > 16) asm volatile("" : "+v"(v[i]));
        RawIO<T>::unpack(v[i], vals);
#pragma unroll
        for (int e = 0; e < VEC; e++) f(vals[e]);
      }
      __builtin_amdgcn_sched_barrier(0);   // one vector's arithmetic at a time: the row itself fills most of the registers
    }
    if (hasTail) f(tailv);
  };
  const A NEG = -r_tmax<A>();
  A mx = NEG;
  sweep([&](A val) { mx = LOG ? (val > mx ? val : mx) : softmax_maxstep<A>(mx, val, clamp); });
  mx = block_allreduce<MaxOp, NT / 64, A>(mx, lds);
  if (!LOG && clamp && mx == NEG) mx = (A)0;
  A sum = (A)0;
  auto term = [&](A val) -> A { if constexpr (LOG) return r_exp<A>(val - mx); else return softmax_term(val, mx, clamp); };
  // fp32 rows: the exponentials take the place of the row in its registers (the same values in the same order of summation);
  // a 16-bit row stays packed and its exponentials are taken again on the way out
  constexpr bool KEEP = sizeof(T) == 4 && sizeof(A) == 4;
  A tailE = tailv;
  if constexpr (KEEP) {
#pragma unroll
    for (int i = 0; i < NV; i++) {
      if ((LongType)i * NT + t < nv) {
        A vals[VEC];
        RawIO<T>::unpack(v[i], vals);
#pragma unroll
        for (int e = 0; e < VEC; e++) { vals[e] = term(vals[e]); sum += vals[e]; }
        v[i] = RawIO<T>::pack(vals);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    if (hasTail) { tailE = term(tailv); sum += tailE; }
  } else {
    sweep([&](A val) { sum += term(val); });
  }
  if constexpr (NT == 64) sum = wave_allreduce<SumOp>(sum); else sum = block_allreduce<SumOp, NT / 64, A>(sum, lds);
  if (!LOG && clamp) sum = sum > (A)1e-6f ? sum : (A)1e-6f;
  // long 16-bit rows: the maximum passes through an opaque copy, so that the exponentials of the sum pass are taken again here
  // instead of being kept in (spilled) registers
  if constexpr (NV > 16 && sizeof(A) == 4 && !KEEP) asm volatile("" : "+v"(mx));
  auto result = [&](A val) -> A {
    const A e = KEEP ? val : term(val);
    if constexpr (LOG) return r_log<A>(e / sum); else return e / sum;
  };
#pragma unroll
  for (int i = 0; i < NV; i++) {
    const LongType iv = (LongType)i * NT + t;
    if (iv < nv) {
      A vals[VEC];
      if constexpr (sizeof(T) == 2 && NV > 16) asm volatile("" : "+v"(v[i]));
      RawIO<T>::unpack(v[i], vals);
#pragma unroll
      for (int e = 0; e < VEC; e++) vals[e] = result(vals[e]);
      const Raw o = RawIO<T>::pack(vals);
      if constexpr (NTS) {   // results of 8 MiB and more: non-temporal, element-aligned 16-byte stores
        nt_store16_elem_aligned(zr + iv * VEC, o);
      } else {
        __builtin_memcpy(zr + iv * VEC, &o, sizeof(Raw));
      }
    }
    __builtin_amdgcn_sched_barrier(0);
  }
  if (hasTail) zr[tail0 + t] = Conv<T>::from(result(tailE));
}
template <typename T, bool LOG>
static bool softmaxBlockRegs(hipStream_t s, const RowArgs& a, const T* x, T* z, int clamp, const RowPlan& p) {
  constexpr LongType V = 16 / sizeof(T);
  if (p.xInner != 1 || p.zInner != 1 || p.rowLen < V || p.rowLen / V > 32 * 512) return false;
  const dim3 grid((unsigned)p.rows), block(512);
  const LongType per = (p.rowLen / V + 511) / 512;
  const bool nts = (size_t)p.rows * (size_t)p.rowLen * sizeof(T) >= ((size_t)8 << 20);
#define SBR(NV) do { if (nts) hipLaunchKernelGGL((softmax_block_regs<T, NV, LOG, true>), grid, block, 0, s, a, x, z, clamp); \
                     else hipLaunchKernelGGL((softmax_block_regs<T, NV, LOG, false>), grid, block, 0, s, a, x, z, clamp); } while (0)
  if (per <= 16) SBR(16); else if (per <= 26) SBR(26); else SBR(32);
#undef SBR
  return true;
}

// many short strided rows (softmax over a non-last axis): one thread per row, neighbouring threads
// own neighbouring rows so that accesses coalesce across the wave
template <typename T>
__global__ __launch_bounds__(256) void softmax_flat(RowArgs a, const T* __restrict__ x, T* __restrict__ z, int clamp) {
  using A = typename Conv<T>::acc;
  const LongType row = (LongType)blockIdx.x * 256 + threadIdx.x;
  if (row >= a.rows) return;
  const LongType xb = walk<LongType>(a.outerX, row), zb = walk<LongType>(a.outerZ, row);
  const A NEG = -r_tmax<A>();
  A mx = NEG;
  for (LongType j = 0; j < a.rowLen; j++) {
    mx = softmax_maxstep<A>(mx, (A)to_float(x[xb + j * a.xInner]), clamp);
  }
  if (clamp && mx == NEG) mx = (A)0;
  A sum = (A)0;
  for (LongType j = 0; j < a.rowLen; j++) sum += softmax_term((A)to_float(x[xb + j * a.xInner]), mx, clamp);
  if (clamp) sum = sum > (A)1e-6f ? sum : (A)1e-6f;
  for (LongType j = 0; j < a.rowLen; j++)
    z[zb + j * a.zInner] = Conv<T>::from(softmax_term((A)to_float(x[xb + j * a.xInner]), mx, clamp) / sum);
}

static RowArgs rowArgs(const RowPlan& p) {
  RowArgs a;
  a.outerX = p.outerX; a.outerZ = p.outerZ; a.rows = p.rows; a.rowLen = p.rowLen; a.xInner = p.xInner; a.zInner = p.zInner;
  return a;
}
static bool rowsVectorOk(const RowPlan& p, const void* x, const void* z, int V) {
  if (p.xInner != 1 || p.zInner != 1 || p.rowLen % V != 0) return false;
  if ((reinterpret_cast<uintptr_t>(x) & 15) || (reinterpret_cast<uintptr_t>(z) & 15)) return false;
  for (int d = 0; d < p.outerX.rank; d++) {
    if (p.outerX.shape[d] > 1 && (p.outerX.stride[d] % V != 0 || p.outerZ.stride[d] % V != 0)) return false;
  }
  return true;
}

template <typename T>
static void softmaxLinear(hipStream_t s, const RowArgs& a, const T* x, T* z, int clamp, int nt) {
  constexpr int V = 16 / sizeof(T);
  const int passes = (int)((a.rowLen / V + 63) / 64);
  // short rows: 8, 16 or 32 lanes per row, so that a wave's loads cover several rows instead of leaving most lanes idle
  // (bf16 rows of 64: 8 of 64 lanes had a vector)
  const LongType lanes = a.rowLen / V;
  if (lanes <= 32) {
#define SG(G) do { const dim3 gg((unsigned)((a.rows + 256 / G - 1) / (256 / G))); \
                   if (nt == 1) hipLaunchKernelGGL((softmax_linear<T, 1, 1, G>), gg, dim3(256), 0, s, a, x, z, clamp); \
                   else if (nt == 2) hipLaunchKernelGGL((softmax_linear<T, 1, 2, G>), gg, dim3(256), 0, s, a, x, z, clamp); \
                   else hipLaunchKernelGGL((softmax_linear<T, 1, 0, G>), gg, dim3(256), 0, s, a, x, z, clamp); } while (0)
    if (lanes <= 8) SG(8); else if (lanes <= 16) SG(16); else SG(32);
#undef SG
    return;
  }
  const dim3 grid((unsigned)((a.rows + 3) / 4));
#define SL(NV) do { if (nt == 1) hipLaunchKernelGGL((softmax_linear<T, NV, 1>), grid, dim3(256), 0, s, a, x, z, clamp); \
                    else if (nt == 2) hipLaunchKernelGGL((softmax_linear<T, NV, 2>), grid, dim3(256), 0, s, a, x, z, clamp); \
                    else hipLaunchKernelGGL((softmax_linear<T, NV, 0>), grid, dim3(256), 0, s, a, x, z, clamp); } while (0)
  switch (passes) {
    case 1: SL(1); break; case 2: SL(2); break; case 3: SL(3); break; case 4: SL(4); break;
    case 5: SL(5); break; case 6: SL(6); break; case 7: SL(7); break; default: SL(8); break;
  }
#undef SL
}
template <>
void softmaxLinear<double>(hipStream_t, const RowArgs&, const double*, double*, int, int) {}

template <typename T>
static void softmaxTyped(hipStream_t s, const void* x, void* z, const RowPlan& p, int clamp) {
  constexpr int V = 16 / sizeof(T);
  RowArgs a = rowArgs(p);
  const T* xt = (const T*)x;
  T* zt = (T*)z;
  const LongType L = p.rowLen;
  if (p.xInner != 1 && p.rows >= 4096 && L <= 4096) {
    hipLaunchKernelGGL((softmax_flat<T>), dim3((unsigned)((p.rows + 255) / 256)), dim3(256), 0, s, a, xt, zt, clamp);
    return;
  }
  const unsigned gw = (unsigned)((p.rows + 3) / 4), gb = (unsigned)p.rows;
  if (rowsVectorOk(p, x, z, V)) {
    const LongType perWave = 64 * V, perBlock = 256 * V;
    // rows streamed once and larger than the last-level cache: non-temporal accesses
    // ... and results of 8 MiB and more through non-temporal stores only (with ordinary stores they sit dirty in the L2
    // until the kernel ends and are flushed then, which the next launch waits for)
    const size_t outBytes = (size_t)p.rows * (size_t)L * sizeof(T);
    const int nt = outBytes * 2 > ((size_t)288 << 20) ? 1 : outBytes >= ((size_t)8 << 20) ? 2 : 0;
    if (sizeof(T) <= 4 && L <= 8 * perWave) {
      softmaxLinear<T>(s, a, xt, zt, clamp, nt);
      return;
    }
#define SM(TPR, NV, GRID) hipLaunchKernelGGL((softmax_rows<T, TPR, NV, V>), dim3(GRID), dim3(256), 0, s, a, xt, zt, clamp, nt)
    if (L <= perWave) { SM(64, 1, gw); return; }
    if (L <= 2 * perWave) { SM(64, 2, gw); return; }
    if (L <= 4 * perWave) { SM(64, 4, gw); return; }
    if (L <= 4 * perBlock && p.rows < 2048) { SM(256, 4, gb); return; }   // few rows: spread each over a block
    if (L <= 8 * perWave) { SM(64, 8, gw); return; }
    if (L <= 4 * perBlock) { SM(256, 4, gb); return; }
    if (L <= 8 * perBlock) { SM(256, 8, gb); return; }
#undef SM
  } else {
    // unit-stride rows that start anywhere or have any length: a wave per row, the row in registers through element-aligned
    // 16-byte loads, the last L % V values one per lane (warm bf16 [192, 1001, 1001]: 2.4 TB/s with one element per load)
    if constexpr (sizeof(T) == 2) {   // (fp32 rows are as fast with one 4-byte element per load: [192, 1023, 1023] 0.293 against 0.307 ms)
      if (p.xInner == 1 && p.zInner == 1 && L >= 2 * V && L / V <= 64 * 16) {
        const LongType per = (L / V + 63) / 64;
        const bool nts = (size_t)p.rows * (size_t)L * sizeof(T) >= ((size_t)8 << 20);
#define SWR(NV) do { if (nts) hipLaunchKernelGGL((softmax_block_regs<T, NV, false, true, 64>), dim3(gw), dim3(256), 0, s, a, xt, zt, clamp); \
                     else hipLaunchKernelGGL((softmax_block_regs<T, NV, false, false, 64>), dim3(gw), dim3(256), 0, s, a, xt, zt, clamp); } while (0)
        if (per <= 2) SWR(2); else if (per <= 4) SWR(4); else if (per <= 8) SWR(8); else SWR(16);
#undef SWR
        return;
      }
    }
    if (L <= 64 * 16) { hipLaunchKernelGGL((softmax_rows<T, 64, 16, 1>), dim3(gw), dim3(256), 0, s, a, xt, zt, clamp, 0); return; }
    if (L <= 256 * 32) { hipLaunchKernelGGL((softmax_rows<T, 256, 32, 1>), dim3(gb), dim3(256), 0, s, a, xt, zt, clamp, 0); return; }
  }
  if constexpr (sizeof(T) <= 4) {
    if (softmaxBlockRegs<T, false>(s, a, xt, zt, clamp, p)) return;
  }
  // unit-stride rows whose x and z starts sit at the same offset from a 16-byte boundary in every row
  if constexpr (sizeof(T) <= 4) {
    constexpr LongType V = 16 / sizeof(T);
    bool same = p.xInner == 1 && p.zInner == 1 && ((reinterpret_cast<uintptr_t>(x) ^ reinterpret_cast<uintptr_t>(z)) & 15) == 0 && p.outerX.rank == p.outerZ.rank;
    for (int d = 0; same && d < p.outerX.rank; d++)
      if (p.outerX.shape[d] > 1 && (p.outerX.stride[d] - p.outerZ.stride[d]) % V != 0) same = false;
    if (same) {
      hipLaunchKernelGGL((softmax_long_vec<T>), dim3(gb), dim3(1024), 0, s, a, xt, zt, clamp);
      return;
    }
  }
  hipLaunchKernelGGL((softmax_long<T>), dim3(gb), dim3(256), 0, s, a, xt, zt, clamp);
}

void launchSoftmax(hipStream_t s, DataType dt, const void* x, void* z, const RowPlan& p, bool clampMode) {
  if (p.rows == 0 || p.rowLen == 0) return;
  ND4J_REQUIRE(p.rows < (1LL << 31), "softmax: too many rows");
  switch (dt) {
    case FLOAT32: softmaxTyped<float>(s, x, z, p, clampMode); break;
    case DOUBLE: softmaxTyped<double>(s, x, z, p, clampMode); break;
    case HALF: softmaxTyped<f16_t>(s, x, z, p, clampMode); break;
    case BFLOAT16: softmaxTyped<bf16_t>(s, x, z, p, clampMode); break;
    default: ND4J_THROW("softmax: unsupported dtype");
  }
  HIP_CHECK(hipGetLastError());
}

// ---- log_softmax ---------------------------------------------------------------------------------------------------------------
// generic/nn/logSoftmax.cpp:34-49 -> helpers/cpu/activations.cpp:100-145,236-256: max, exp(x - max), sum, divide, log, in
// that order (a term whose exponential underflows comes out as -inf, as it does there).  One block per row, three passes;
// rows and inner strides are arbitrary.  Not a tuned kernel.
template <typename T>
__global__ __launch_bounds__(256) void log_softmax_rows(RowArgs a, const T* __restrict__ x, T* __restrict__ z) {
  using A = typename Conv<T>::acc;
  __shared__ A lds[4];
  const LongType row = blockIdx.x;
  const LongType xb = walk<LongType>(a.outerX, row), zb = walk<LongType>(a.outerZ, row);
  A mx = -r_tmax<A>();
  for (LongType j = threadIdx.x; j < a.rowLen; j += 256) { const A v = (A)to_float(x[xb + j * a.xInner]); mx = v > mx ? v : mx; }
  mx = block_allreduce<MaxOp, 4, A>(mx, lds);
  A sum = (A)0;
  for (LongType j = threadIdx.x; j < a.rowLen; j += 256) sum += r_exp<A>((A)to_float(x[xb + j * a.xInner]) - mx);
  sum = block_allreduce<SumOp, 4, A>(sum, lds);
  for (LongType j = threadIdx.x; j < a.rowLen; j += 256)
    z[zb + j * a.zInner] = Conv<T>::from(r_log<A>(r_exp<A>((A)to_float(x[xb + j * a.xInner]) - mx) / sum));
}
void launchLogSoftmax(hipStream_t s, DataType dt, const void* x, void* z, const RowPlan& p) {
  if (p.rows == 0 || p.rowLen == 0) return;
  ND4J_REQUIRE(p.rows < (1LL << 31), "log_softmax: too many rows");
  RowArgs a = rowArgs(p);
  const dim3 g((unsigned)p.rows), b(256);
  // long unit-stride rows whose x and z starts sit at the same offset from a 16-byte boundary: the vector kernel of the
  // long-row softmax with the logarithm on the way out
  if (p.rowLen >= 8192) {
    bool done = false;
    if (dt == FLOAT32) done = softmaxBlockRegs<float, true>(s, a, (const float*)x, (float*)z, 0, p);
    else if (dt == HALF) done = softmaxBlockRegs<f16_t, true>(s, a, (const f16_t*)x, (f16_t*)z, 0, p);
    else if (dt == BFLOAT16) done = softmaxBlockRegs<bf16_t, true>(s, a, (const bf16_t*)x, (bf16_t*)z, 0, p);
    if (done) { HIP_CHECK(hipGetLastError()); return; }
  }
  if ((dt == FLOAT32 || dt == HALF || dt == BFLOAT16) && p.rowLen >= 8192 && p.xInner == 1 && p.zInner == 1 &&
      ((reinterpret_cast<uintptr_t>(x) ^ reinterpret_cast<uintptr_t>(z)) & 15) == 0 && p.outerX.rank == p.outerZ.rank) {
    const LongType V = dt == FLOAT32 ? 4 : 8;
    bool same = true;
    for (int d = 0; same && d < p.outerX.rank; d++)
      if (p.outerX.shape[d] > 1 && (p.outerX.stride[d] - p.outerZ.stride[d]) % V != 0) same = false;
    if (same) {
      if (dt == FLOAT32) hipLaunchKernelGGL((softmax_long_vec<float, true>), g, dim3(1024), 0, s, a, (const float*)x, (float*)z, 0);
      else if (dt == HALF) hipLaunchKernelGGL((softmax_long_vec<f16_t, true>), g, dim3(1024), 0, s, a, (const f16_t*)x, (f16_t*)z, 0);
      else hipLaunchKernelGGL((softmax_long_vec<bf16_t, true>), g, dim3(1024), 0, s, a, (const bf16_t*)x, (bf16_t*)z, 0);
      HIP_CHECK(hipGetLastError());
      return;
    }
  }
  switch (dt) {
    case FLOAT32: hipLaunchKernelGGL((log_softmax_rows<float>), g, b, 0, s, a, (const float*)x, (float*)z); break;
    case DOUBLE: hipLaunchKernelGGL((log_softmax_rows<double>), g, b, 0, s, a, (const double*)x, (double*)z); break;
    case HALF: hipLaunchKernelGGL((log_softmax_rows<f16_t>), g, b, 0, s, a, (const f16_t*)x, (f16_t*)z); break;
    case BFLOAT16: hipLaunchKernelGGL((log_softmax_rows<bf16_t>), g, b, 0, s, a, (const bf16_t*)x, (bf16_t*)z); break;
    default: ND4J_THROW("log_softmax: unsupported dtype");
  }
  HIP_CHECK(hipGetLastError());
}

// ---- layer_norm -------------------------------------------------------------------------------------------
template <typename A> __device__ __forceinline__ A r_sqrt(A x);
template <> __device__ __forceinline__ float r_sqrt<float>(float x) { return sqrtf(x); }
template <> __device__ __forceinline__ double r_sqrt<double>(double x) { return sqrt(x); }

template <typename T, int TPR, int NV, int VEC>
__global__ __launch_bounds__(256) void layernorm_rows(RowArgs a, const T* __restrict__ x, const T* __restrict__ gain,
                                                      const T* __restrict__ bias, T* __restrict__ z, float eps) {
  using A = typename Conv<T>::acc;
  using VT = Vec<T, VEC>;
  constexpr int ROWS = 256 / TPR;
  __shared__ A lds[4];
  const int t = threadIdx.x % TPR;
  LongType row = (LongType)blockIdx.x * ROWS + threadIdx.x / TPR;
  const bool live = row < a.rows;
  if (!live) row = a.rows - 1;
  const LongType xb = walk<LongType>(a.outerX, row), zb = walk<LongType>(a.outerZ, row);
  const LongType L = a.rowLen;
  A vals[NV * VEC];
  A sum = (A)0;
  // vector rows (L a multiple of VEC, so at least one whole vector): every load is issued unconditionally, past the row's end
  // on its last vector, so that the row costs one trip to memory and not one per vector
  typename RawIO<T>::raw xraw[VEC > 1 ? NV : 1];
  if (VEC > 1) {
#pragma unroll
    for (int i = 0; i < NV; i++) {
      const LongType e0 = ((LongType)t + (LongType)i * TPR) * VEC;
      xraw[VEC > 1 ? i : 0] = *reinterpret_cast<const typename RawIO<T>::raw*>(x + xb + (e0 < L ? e0 : L - VEC));
    }
  }
#pragma unroll
  for (int i = 0; i < NV; i++) {
    const LongType e0 = ((LongType)t + (LongType)i * TPR) * VEC;
    if (VEC > 1) {
      if (e0 < L) {
        RawIO<T>::unpack(xraw[VEC > 1 ? i : 0], &vals[i * VEC]);
#pragma unroll
        for (int e = 0; e < VEC; e++) sum += vals[i * VEC + e];
      } else {
#pragma unroll
        for (int e = 0; e < VEC; e++) vals[i * VEC + e] = (A)0;
      }
    } else {
      vals[i] = e0 < L ? (A)to_float(x[xb + e0 * a.xInner]) : (A)0;
      sum += vals[i];
    }
  }
  sum = row_allreduce<SumOp, TPR, A>(sum, lds);
  const A mean = sum / (A)L;
  A sq = (A)0;
#pragma unroll
  for (int i = 0; i < NV; i++) {
    const LongType e0 = ((LongType)t + (LongType)i * TPR) * VEC;
#pragma unroll
    for (int e = 0; e < VEC; e++) if (e0 + e < L) { A d = vals[i * VEC + e] - mean; sq += d * d; }
  }
  sq = row_allreduce<SumOp, TPR, A>(sq, lds);
  const A var = L > 1 ? sq / (A)L : (A)0;
  const A rstd = (A)1 / r_sqrt<A>(var + (A)eps);   // one division per row
  if (!live) return;
  typename RawIO<T>::raw graw[VEC > 1 ? NV : 1], braw[VEC > 1 ? NV : 1];
  if (VEC > 1) {   // gain and bias the same way: all loads before the first use
#pragma unroll
    for (int i = 0; i < NV; i++) {
      const LongType e0 = ((LongType)t + (LongType)i * TPR) * VEC;
      const LongType ec = e0 < L ? e0 : L - VEC;
      graw[VEC > 1 ? i : 0] = *reinterpret_cast<const typename RawIO<T>::raw*>(gain + ec);
      braw[VEC > 1 ? i : 0] = bias ? *reinterpret_cast<const typename RawIO<T>::raw*>(bias + ec) : graw[VEC > 1 ? i : 0];
    }
  }
#pragma unroll
  for (int i = 0; i < NV; i++) {
    const LongType e0 = ((LongType)t + (LongType)i * TPR) * VEC;
    if (e0 >= L) continue;
    if (VEC > 1) {
      A g[VEC], b[VEC];
      RawIO<T>::unpack(graw[VEC > 1 ? i : 0], g);
      if (bias) RawIO<T>::unpack(braw[VEC > 1 ? i : 0], b);
#pragma unroll
      for (int e = 0; e < VEC; e++) {
        A y = (vals[i * VEC + e] - mean) * rstd * g[e];
        if (bias) y += b[e];
        vals[i * VEC + e] = y;
      }
      *reinterpret_cast<typename RawIO<T>::raw*>(z + zb + e0) = RawIO<T>::pack(&vals[i * VEC]);
    } else {
      A y = (vals[i] - mean) * rstd * (A)to_float(gain[e0]);
      if (bias) y += (A)to_float(bias[e0]);
      z[zb + e0 * a.zInner] = Conv<T>::from(y);
    }
  }
}

// One wave per row for rows at a constant pitch (the usual case: a dense or row-strided matrix), vector path only.
// No shape walk and no predicated loads: every lane issues its x / gain / bias vectors at once (lanes past the row's
// end re-read the last vector and are masked out of the sums), so the three latencies overlap instead of queueing.
// ADD: the row normalised is x + addend, rounded through the storage type and also written to sumOut -- a pairwise Add
// followed by layer_norm on its result, in one pass (sumOut may be x itself: a wave reads a row before it writes it).
// G: lanes per row (64: a wave per row; 8, 16, 32 with NV == 1 and RPW == 1: several short rows per wave)
template <typename T, int NV, bool HAS_BIAS, int RPW, bool ADD = false, int G = 64>
__global__ __launch_bounds__(256) void layernorm_linear(const T* __restrict__ x, const T* __restrict__ gain, const T* __restrict__ bias,
                                                        T* __restrict__ z, LongType rows, int L, LongType xPitch, LongType zPitch, float eps,
                                                        const T* addend = nullptr, LongType aPitch = 0, T* sumOut = nullptr, LongType sPitch = 0,
                                                        int nts = 0) {   // nts: the result through non-temporal stores (8 MiB and more)
  using A = typename Conv<T>::acc;
  using Raw = typename RawIO<T>::raw;
  constexpr int VEC = RawIO<T>::N;
  const int t = threadIdx.x & (G - 1);
  // a wave owns RPW consecutive rows: gain and bias are fetched once for all of them
  const LongType row0 = ((LongType)blockIdx.x * (256 / G) + threadIdx.x / G) * RPW;
  if (row0 >= rows) return;
  int e0[NV];
  A keep[NV];
  Raw xv[RPW][NV], gv[NV], bv[NV], av[ADD ? RPW : 1][ADD ? NV : 1];
#pragma unroll
  for (int i = 0; i < NV; i++) {
    const int e = (t + i * G) * VEC;
    keep[i] = e < L ? (A)1 : (A)0;
    e0[i] = e < L ? e : L - VEC;
  }
#pragma unroll
  for (int r = 0; r < RPW; r++) {
    const LongType row = row0 + r < rows ? row0 + r : rows - 1;
#pragma unroll
    for (int i = 0; i < NV; i++) {
      xv[r][i] = *reinterpret_cast<const Raw*>(x + row * xPitch + e0[i]);
      if (ADD) av[ADD ? r : 0][ADD ? i : 0] = *reinterpret_cast<const Raw*>(addend + row * aPitch + e0[i]);
    }
  }
#pragma unroll
  for (int i = 0; i < NV; i++) {
    gv[i] = *reinterpret_cast<const Raw*>(gain + e0[i]);
    if (HAS_BIAS) bv[i] = *reinterpret_cast<const Raw*>(bias + e0[i]);
  }
  // a lone row (a decode step) waits on gain and bias coming cold from HBM: one empty asm that "uses" every loaded
  // vector makes the compiler issue all the loads ahead of it, instead of sinking gain and bias below the row's first
  // reduction (a second trip to memory)
  if (RPW == 1) {
    if (!HAS_BIAS) {
#pragma unroll
      for (int i = 0; i < NV; i++) bv[i] = gv[i];
    }
    if (NV == 1) asm volatile("" : "+v"(xv[0][0]), "+v"(gv[0]), "+v"(bv[0]));
    if (NV == 2) asm volatile("" : "+v"(xv[0][0]), "+v"(xv[0][NV > 1 ? 1 : 0]), "+v"(gv[0]), "+v"(gv[NV > 1 ? 1 : 0]), "+v"(bv[0]), "+v"(bv[NV > 1 ? 1 : 0]));
    if (NV == 3) asm volatile("" : "+v"(xv[0][0]), "+v"(xv[0][NV > 1 ? 1 : 0]), "+v"(xv[0][NV > 2 ? 2 : 0]), "+v"(gv[0]), "+v"(gv[NV > 1 ? 1 : 0]), "+v"(gv[NV > 2 ? 2 : 0]),
                                    "+v"(bv[0]), "+v"(bv[NV > 1 ? 1 : 0]), "+v"(bv[NV > 2 ? 2 : 0]));
    if (NV == 4) asm volatile("" : "+v"(xv[0][0]), "+v"(xv[0][NV > 1 ? 1 : 0]), "+v"(xv[0][NV > 2 ? 2 : 0]), "+v"(xv[0][NV > 3 ? 3 : 0]), "+v"(gv[0]), "+v"(gv[NV > 1 ? 1 : 0]),
                                    "+v"(gv[NV > 2 ? 2 : 0]), "+v"(gv[NV > 3 ? 3 : 0]), "+v"(bv[0]), "+v"(bv[NV > 1 ? 1 : 0]), "+v"(bv[NV > 2 ? 2 : 0]), "+v"(bv[NV > 3 ? 3 : 0]));
  }
  A vals[RPW][NV * VEC];
  if (RPW == 1) {
    // one row per wave: the shared row routine (also what a product that normalises its input row runs)
#pragma unroll
    for (int i = 0; i < NV; i++) {
      RawIO<T>::unpack(xv[0][i], &vals[0][i * VEC]);
      if (ADD) {
        A add[VEC];
        RawIO<T>::unpack(av[0][ADD ? i : 0], add);
#pragma unroll
        for (int e = 0; e < VEC; e++) vals[0][i * VEC + e] += add[e];
        const Raw packed = RawIO<T>::pack(&vals[0][i * VEC]);   // the sum as the separate Add would have stored it
        if (keep[i] != (A)0) *reinterpret_cast<Raw*>(sumOut + row0 * sPitch + e0[i]) = packed;
        RawIO<T>::unpack(packed, &vals[0][i * VEC]);
      }
    }
    ln_wave_row<T, NV, HAS_BIAS, G>(vals[0], gv, bv, keep, L, eps);
    T* zr = z + row0 * zPitch;
#pragma unroll
    for (int i = 0; i < NV; i++)
      if (keep[i] != (A)0) store_vec(reinterpret_cast<Raw*>(zr + e0[i]), RawIO<T>::pack(&vals[0][i * VEC]), nts != 0);
    return;
  }
  A sum[RPW];
#pragma unroll
  for (int r = 0; r < RPW; r++) {
    sum[r] = (A)0;
#pragma unroll
    for (int i = 0; i < NV; i++) {
      RawIO<T>::unpack(xv[r][i], &vals[r][i * VEC]);
      A part = (A)0;
#pragma unroll
      for (int e = 0; e < VEC; e++) part += vals[r][i * VEC + e];
      sum[r] += part * keep[i];
    }
  }
#pragma unroll
  for (int r = 0; r < RPW; r++) sum[r] = wave_allreduce<SumOp>(sum[r]);
  A sq[RPW];
#pragma unroll
  for (int r = 0; r < RPW; r++) {
    const A mean = sum[r] / (A)L;
    sq[r] = (A)0;
#pragma unroll
    for (int i = 0; i < NV; i++) {
      A part = (A)0;
#pragma unroll
      for (int e = 0; e < VEC; e++) { const A d = vals[r][i * VEC + e] - mean; vals[r][i * VEC + e] = d; part += d * d; }
      sq[r] += part * keep[i];
    }
  }
#pragma unroll
  for (int r = 0; r < RPW; r++) sq[r] = wave_allreduce<SumOp>(sq[r]);
#pragma unroll
  for (int r = 0; r < RPW; r++) {
    if (row0 + r >= rows) break;
    const A var = L > 1 ? sq[r] / (A)L : (A)0;
    const A rstd = (A)1 / r_sqrt<A>(var + (A)eps);
    T* zr = z + (row0 + r) * zPitch;
#pragma unroll
    for (int i = 0; i < NV; i++) {
      A g[VEC], b[VEC];
      RawIO<T>::unpack(gv[i], g);
      if (HAS_BIAS) RawIO<T>::unpack(bv[i], b);
#pragma unroll
      for (int e = 0; e < VEC; e++) {
        A y = vals[r][i * VEC + e] * rstd * g[e];
        if (HAS_BIAS) y += b[e];
        vals[r][i * VEC + e] = y;
      }
      if (keep[i] != (A)0) store_vec(reinterpret_cast<Raw*>(zr + e0[i]), RawIO<T>::pack(&vals[r][i * VEC]), nts != 0);
    }
  }
}

// a result vector on its way out: through a non-temporal store when the host asks for it (results of 8 MiB and more:
// written with ordinary stores they sit dirty in the L2 until the kernel ends and are flushed then, which the next launch
// waits for), else an ordinary one
template <bool NTS, typename Raw>
__device__ __forceinline__ void store_row_vec(Raw* p, const Raw& v) {
  if constexpr (!NTS) {
    *p = v;
  } else if constexpr (sizeof(Raw) == 12) {
    typedef unsigned u32x3a __attribute__((ext_vector_type(3), aligned(4)));
    const u32x3a t = {v[0], v[1], v[2]};
    __builtin_nontemporal_store(t, reinterpret_cast<u32x3a*>(p));
  } else {
    __builtin_nontemporal_store(v, p);
  }
}

// Many rows: two consecutive rows per wave, gain and bias fetched once for both, every load of the pair issued before
// the first use.  The grid normally gives every wave one pair; beyond 2^20 blocks a wave walks on to pair pr + W with
// that pair's loads issued ahead.  (About ten vector instructions per element: a 16-bit row is as much arithmetic as an
// fp32 row of the same length in half the bytes, which is why bf16 [16384, 768] takes 9.5 us where gelu takes 5.3.)
template <typename T, int NV, bool HAS_BIAS, typename IO = RawIO<T>, bool WALK = true, bool NTS = false>
__global__ __launch_bounds__(256, WALK ? 1 : 8) void layernorm_stream(const T* __restrict__ x, const T* __restrict__ gain, const T* __restrict__ bias, T* __restrict__ z,
                                                        LongType rows, int L, LongType xPitch, LongType zPitch, float eps) {
  using A = typename Conv<T>::acc;
  using Raw = typename IO::raw;
  constexpr int VEC = IO::N;
  const int t = threadIdx.x & 63;
  const LongType W = (LongType)gridDim.x * 4, pairs = (rows + 1) / 2;
  LongType pr = (LongType)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (pr >= pairs) return;
  int e0[NV];
  A keep[NV];
#pragma unroll
  for (int i = 0; i < NV; i++) {
    const int e = (t + i * 64) * VEC;
    keep[i] = e < L ? (A)1 : (A)0;
    e0[i] = e < L ? e : L - VEC;
  }
  Raw cur[2][NV], nxt[2][NV], gv[NV], bv[NV];
  auto load = [&](LongType pair, Raw (&dst)[2][NV]) {
#pragma unroll
    for (int r = 0; r < 2; r++) {
      const LongType row = 2 * pair + r < rows ? 2 * pair + r : rows - 1;
#pragma unroll
      for (int i = 0; i < NV; i++) dst[r][i] = *reinterpret_cast<const Raw*>(x + row * xPitch + e0[i]);
    }
  };
  load(pr, cur);
  auto loadGainBias = [&]() {
#pragma unroll
    for (int i = 0; i < NV; i++) {
      gv[i] = *reinterpret_cast<const Raw*>(gain + e0[i]);
      if (HAS_BIAS) bv[i] = *reinterpret_cast<const Raw*>(bias + e0[i]);
    }
  };
  loadGainBias();
  for (; pr < pairs; pr += W) {
    const bool more = WALK && pr + W < pairs;
    if (more) load(pr + W, nxt);
    A vals[2][NV * VEC], sum[2];
#pragma unroll
    for (int r = 0; r < 2; r++) {
      sum[r] = (A)0;
#pragma unroll
      for (int i = 0; i < NV; i++) {
        IO::unpack(cur[r][i], &vals[r][i * VEC]);
        A part = (A)0;
#pragma unroll
        for (int e = 0; e < VEC; e++) part += vals[r][i * VEC + e];
        sum[r] += part * keep[i];
      }
    }
#pragma unroll
    for (int r = 0; r < 2; r++) sum[r] = wave_allreduce<SumOp>(sum[r]);
    A sq[2];
#pragma unroll
    for (int r = 0; r < 2; r++) {
      const A mean = sum[r] / (A)L;
      sq[r] = (A)0;
#pragma unroll
      for (int i = 0; i < NV; i++) {
        A part = (A)0;
#pragma unroll
        for (int e = 0; e < VEC; e++) { const A d = vals[r][i * VEC + e] - mean; vals[r][i * VEC + e] = d; part += d * d; }
        sq[r] += part * keep[i];
      }
    }
#pragma unroll
    for (int r = 0; r < 2; r++) sq[r] = wave_allreduce<SumOp>(sq[r]);
#pragma unroll
    for (int r = 0; r < 2; r++) {
      if (2 * pr + r >= rows) break;
      const A var = L > 1 ? sq[r] / (A)L : (A)0;
      const A rstd = (A)1 / r_sqrt<A>(var + (A)eps);
      T* zr = z + (2 * pr + r) * zPitch;
#pragma unroll
      for (int i = 0; i < NV; i++) {
        A g[VEC], b[VEC];
        IO::unpack(gv[i], g);
        if (HAS_BIAS) IO::unpack(bv[i], b);
#pragma unroll
        for (int e = 0; e < VEC; e++) {
          A y = vals[r][i * VEC + e] * rstd * g[e];
          if (HAS_BIAS) y += b[e];
          vals[r][i * VEC + e] = y;
        }
        if (keep[i] != (A)0) store_row_vec<NTS>(reinterpret_cast<Raw*>(zr + e0[i]), IO::pack(&vals[r][i * VEC]));
      }
    }
    if (!WALK) break;
    if (more) {
#pragma unroll
      for (int r = 0; r < 2; r++)
#pragma unroll
        for (int i = 0; i < NV; i++) cur[r][i] = nxt[r][i];
    }
  }
}

// Rows too long for a block's registers (beyond 8 vectors per thread): one block of 16 waves per row and three passes over
// it with 16-byte vectors -- total, squared distances, output; the second and third find the row in the L2.
template <typename T, bool HAS_BIAS>
__global__ __launch_bounds__(1024) void layernorm_long(const T* __restrict__ x, const T* __restrict__ gain, const T* __restrict__ bias, T* __restrict__ z,
                                                       LongType L, LongType xPitch, LongType zPitch, float eps) {
  using A = typename Conv<T>::acc;
  using IO = RawIO<T>;
  using Raw = typename IO::raw;
  constexpr int VEC = IO::N;
  __shared__ A lds[16];
  const T* xr = x + (LongType)blockIdx.x * xPitch;
  T* zr = z + (LongType)blockIdx.x * zPitch;
  const LongType nv = L / VEC;
  constexpr int U = 4;   // vectors a thread has in flight (positions past the row's end re-read its last vector and are left out)
  A sum = (A)0;
  for (LongType v0 = threadIdx.x; v0 < nv; v0 += U * 1024) {
    Raw r[U];
#pragma unroll
    for (int u = 0; u < U; u++) { const LongType v = v0 + u * 1024; r[u] = *reinterpret_cast<const Raw*>(xr + (v < nv ? v : nv - 1) * VEC); }
#pragma unroll
    for (int u = 0; u < U; u++) {
      A vals[VEC];
      IO::unpack(r[u], vals);
      A part = (A)0;
#pragma unroll
      for (int e = 0; e < VEC; e++) part += vals[e];
      if (v0 + u * 1024 < nv) sum += part;
    }
  }
  sum = block_allreduce<SumOp, 16, A>(sum, lds);
  const A mean = sum / (A)L;
  A sq = (A)0;
  for (LongType v0 = threadIdx.x; v0 < nv; v0 += U * 1024) {
    Raw r[U];
#pragma unroll
    for (int u = 0; u < U; u++) { const LongType v = v0 + u * 1024; r[u] = *reinterpret_cast<const Raw*>(xr + (v < nv ? v : nv - 1) * VEC); }
#pragma unroll
    for (int u = 0; u < U; u++) {
      A vals[VEC];
      IO::unpack(r[u], vals);
      A part = (A)0;
#pragma unroll
      for (int e = 0; e < VEC; e++) { const A d = vals[e] - mean; part += d * d; }
      if (v0 + u * 1024 < nv) sq += part;
    }
  }
  sq = block_allreduce<SumOp, 16, A>(sq, lds);
  const A var = L > 1 ? sq / (A)L : (A)0;
  const A rstd = (A)1 / r_sqrt<A>(var + (A)eps);
  for (LongType v0 = threadIdx.x; v0 < nv; v0 += 2 * 1024) {
    Raw r[2], gr[2], br[2];
#pragma unroll
    for (int u = 0; u < 2; u++) {
      const LongType v = v0 + u * 1024, vc = v < nv ? v : nv - 1;
      r[u] = *reinterpret_cast<const Raw*>(xr + vc * VEC);
      gr[u] = *reinterpret_cast<const Raw*>(gain + vc * VEC);
      if (HAS_BIAS) br[u] = *reinterpret_cast<const Raw*>(bias + vc * VEC);
    }
#pragma unroll
    for (int u = 0; u < 2; u++) {
      A vals[VEC], g[VEC], b[VEC];
      IO::unpack(r[u], vals);
      IO::unpack(gr[u], g);
      if (HAS_BIAS) IO::unpack(br[u], b);
#pragma unroll
      for (int e = 0; e < VEC; e++) {
        A y = (vals[e] - mean) * rstd * g[e];
        if (HAS_BIAS) y += b[e];
        vals[e] = y;
      }
      if (v0 + u * 1024 < nv) *reinterpret_cast<Raw*>(zr + (v0 + u * 1024) * VEC) = IO::pack(vals);
    }
  }
}

// One wave per row for unit-stride rows at a constant pitch that the aligned vector kernels cannot take -- a row length that is
// not a whole number of 16-byte vectors (770), rows, gain or bias that start off 16-byte boundaries: element-aligned 16-byte
// loads (global memory runs in unaligned access mode), the last L % VEC values one per lane, the row in registers.  Same
// arithmetic as ln_wave_row.  (These rows used to go one element per load: warm bf16 [16000, 770] 2.0 TB/s.)
template <typename T, int NV, bool HAS_BIAS, bool NTS>
__global__ __launch_bounds__(256) void layernorm_wave_regs(const T* __restrict__ x, const T* __restrict__ gain, const T* __restrict__ bias,
                                                           T* __restrict__ z, LongType rows, int L, LongType xPitch, LongType zPitch, float eps) {
  using A = typename Conv<T>::acc;
  using Raw = typename RawIO<T>::raw;
  constexpr int VEC = RawIO<T>::N;
  const int lane = threadIdx.x & 63;
  const LongType row = (LongType)blockIdx.x * 4 + threadIdx.x / 64;
  if (row >= rows) return;
  const T* xr = x + row * xPitch;
  T* zr = z + row * zPitch;
  const int nv = L / VEC, tail0 = nv * VEC;
  Raw xv[NV], gv[NV], bv[NV];
#pragma unroll
  for (int i = 0; i < NV; i++) {
    const int iv = i * 64 + lane, c = (iv < nv ? iv : nv - 1) * VEC;
    __builtin_memcpy(&xv[i], xr + c, sizeof(Raw));
    __builtin_memcpy(&gv[i], gain + c, sizeof(Raw));
    if (HAS_BIAS) __builtin_memcpy(&bv[i], bias + c, sizeof(Raw));
  }
  const bool hasTail = tail0 + lane < L;
  const int te = hasTail ? tail0 + lane : 0;
  A tx = hasTail ? (A)to_float(xr[te]) : (A)0;
  const A tg = (A)to_float(gain[te]), tb = HAS_BIAS ? (A)to_float(bias[te]) : (A)0;
  A vals[NV][VEC];
  A sum = (A)0;
#pragma unroll
  for (int i = 0; i < NV; i++) {
    RawIO<T>::unpack(xv[i], vals[i]);
    A part = (A)0;
#pragma unroll
    for (int e = 0; e < VEC; e++) part += vals[i][e];
    sum += i * 64 + lane < nv ? part : (A)0;
  }
  sum += tx;
  sum = wave_allreduce<SumOp>(sum);
  const A mean = sum / (A)L;
  A sq = (A)0;
#pragma unroll
  for (int i = 0; i < NV; i++) {
    A part = (A)0;
#pragma unroll
    for (int e = 0; e < VEC; e++) { const A d = vals[i][e] - mean; vals[i][e] = d; part += d * d; }
    sq += i * 64 + lane < nv ? part : (A)0;
  }
  tx -= mean;
  sq += hasTail ? tx * tx : (A)0;
  sq = wave_allreduce<SumOp>(sq);
  const A var = L > 1 ? sq / (A)L : (A)0;
  const A rstd = (A)1 / (A)sqrtf((float)(var + (A)eps));
#pragma unroll
  for (int i = 0; i < NV; i++) {
    const int iv = i * 64 + lane;
    if (iv < nv) {
      A g[VEC], b[VEC];
      RawIO<T>::unpack(gv[i], g);
      if (HAS_BIAS) RawIO<T>::unpack(bv[i], b);
#pragma unroll
      for (int e = 0; e < VEC; e++) {
        A y = vals[i][e] * rstd * g[e];
        if (HAS_BIAS) y += b[e];
        vals[i][e] = y;
      }
      const Raw o = RawIO<T>::pack(vals[i]);
      if constexpr (NTS) nt_store16_elem_aligned(zr + iv * VEC, o);
      else __builtin_memcpy(zr + iv * VEC, &o, sizeof(Raw));
    }
  }
  if (hasTail) {
    A y = tx * rstd * tg;
    if (HAS_BIAS) y += tb;
    zr[te] = Conv<T>::from(y);
  }
}
template <typename T>
static bool layerNormTyped(hipStream_t s, const void* x, const void* gain, const void* bias, void* z, const RowPlan& p, float eps) {
  constexpr int V = 16 / sizeof(T);
  RowArgs a = rowArgs(p);
  const T* xt = (const T*)x; const T* gt = (const T*)gain; const T* bt = (const T*)bias; T* zt = (T*)z;
  const LongType L = p.rowLen;
  const unsigned gw = (unsigned)((p.rows + 3) / 4), gb = (unsigned)p.rows;
  bool vec = rowsVectorOk(p, x, z, V) && (reinterpret_cast<uintptr_t>(gain) & 15) == 0 && (!bias || (reinterpret_cast<uintptr_t>(bias) & 15) == 0);
  if (vec) {
    const LongType perWave = 64 * V, perBlock = 256 * V;
#define LN(TPR, NV, GRID) hipLaunchKernelGGL((layernorm_rows<T, TPR, NV, V>), dim3(GRID), dim3(256), 0, s, a, xt, gt, bt, zt, eps)
    // rows at a constant pitch that fit one wave
    const bool linear = p.outerX.rank <= 1 && p.outerZ.rank <= 1 && L < (1 << 30);
    if (linear && L <= 8 * perWave) {
      const LongType xp = p.outerX.rank ? p.outerX.stride[0] : 0, zp = p.outerZ.rank ? p.outerZ.stride[0] : 0;
      // many rows: two per wave (layernorm_stream: gain and bias fetched once for both); few rows: one per wave, so that every CU gets some
      const bool pair = p.rows >= 4096 && L <= 4 * perWave;
      const int ntsL = (size_t)p.rows * (size_t)L * sizeof(T) >= ((size_t)8 << 20) ? 1 : 0;   // see store_row_vec
#define LNL(NV) do { if (bt) hipLaunchKernelGGL((layernorm_linear<T, NV, true, 1>), dim3(gw), dim3(256), 0, s, xt, gt, bt, zt, p.rows, (int)L, xp, zp, eps, (const T*)nullptr, (LongType)0, (T*)nullptr, (LongType)0, ntsL); \
                     else hipLaunchKernelGGL((layernorm_linear<T, NV, false, 1>), dim3(gw), dim3(256), 0, s, xt, gt, bt, zt, p.rows, (int)L, xp, zp, eps, (const T*)nullptr, (LongType)0, (T*)nullptr, (LongType)0, ntsL); } while (0)
      // short rows: 8, 16 or 32 lanes per row
      if constexpr (sizeof(T) <= 4) {
        const LongType lanes = L / V;
        if (lanes <= 32) {
#define LNG(G) do { const unsigned gg = (unsigned)((p.rows + 256 / G - 1) / (256 / G)); \
                    if (bt) hipLaunchKernelGGL((layernorm_linear<T, 1, true, 1, false, G>), dim3(gg), dim3(256), 0, s, xt, gt, bt, zt, p.rows, (int)L, xp, zp, eps); \
                    else hipLaunchKernelGGL((layernorm_linear<T, 1, false, 1, false, G>), dim3(gg), dim3(256), 0, s, xt, gt, bt, zt, p.rows, (int)L, xp, zp, eps); } while (0)
          if (lanes <= 8) LNG(8); else if (lanes <= 16) LNG(16); else LNG(32);
#undef LNG
          return true;
        }
      }
      if (pair) {
        // one pair per wave while the grid allows it (fewer, longer-running waves measured slower: bf16 [16384, 768] 12.7 us
        // per launch with one pair per wave, 13.5 with four, 14.1 with eight)
        const unsigned gs = (unsigned)std::min<LongType>((p.rows + 7) / 8, (LongType)1 << 20);
        // every wave has one pair only (12-byte vectors, up to two passes): the variant without the next pair's registers,
        // 59 instead of 93 of them, eight waves per SIMD.  bf16 [16384, 768] 12.7 -> 11.8 us; the same variant of the 16-byte
        // kernels measured equal or slower (bf16 rows of 512 8.8 -> 9.1 us, fp32 rows of 384 12.0 -> 12.6) and is not built
        const bool oneEach = (LongType)gs * 8 >= p.rows;
        // results of 8 MiB and more leave through non-temporal stores (see store_row_vec)
        const bool nts = (size_t)p.rows * (size_t)L * sizeof(T) >= ((size_t)8 << 20);
#define LNS_(NV, B, NTS) hipLaunchKernelGGL((layernorm_stream<T, NV, B, RawIO<T>, true, NTS>), dim3(gs), dim3(256), 0, s, xt, gt, bt, zt, p.rows, (int)L, xp, zp, eps)
#define LNS(NV) do { if (bt) { if (nts) LNS_(NV, true, true); else LNS_(NV, true, false); } \
                     else { if (nts) LNS_(NV, false, true); else LNS_(NV, false, false); } } while (0)
        // 16-bit rows of a whole number of 384-value passes that are not a whole number of 512-value ones (768: one and a
        // half): 12-byte vectors, every load slot used
        if constexpr (sizeof(T) == 2) {
          if (L % 384 == 0 && L % 512 != 0 && L <= 4 * 384) {
#define LNS12_(NV, B, WALK, NTS) hipLaunchKernelGGL((layernorm_stream<T, NV, B, RawIO12<T>, WALK, NTS>), dim3(gs), dim3(256), 0, s, xt, gt, bt, zt, p.rows, (int)L, xp, zp, eps)
#define LNS12W(NV, WALK) do { if (bt) { if (nts) LNS12_(NV, true, WALK, true); else LNS12_(NV, true, WALK, false); } \
                              else { if (nts) LNS12_(NV, false, WALK, true); else LNS12_(NV, false, WALK, false); } } while (0)
#define LNS12(NV) do { if (oneEach && NV <= 2) LNS12W(NV, (NV > 2)); else LNS12W(NV, true); } while (0)
            if (L == 384) LNS12(1); else if (L == 768) LNS12(2); else LNS12(3);
#undef LNS12
#undef LNS12W
#undef LNS12_
            return true;
          }
        }
        if (L <= perWave) LNS(1); else if (L <= 2 * perWave) LNS(2); else if (L <= 3 * perWave) LNS(3); else LNS(4);
#undef LNS
#undef LNS_
        return true;
      }
      if (L <= perWave) { LNL(1); return true; }
      if (L <= 2 * perWave) { LNL(2); return true; }
      if (L <= 3 * perWave) { LNL(3); return true; }   // 768 floats: three full passes, no clamped re-reads
      if (L <= 4 * perWave) { LNL(4); return true; }
      // up to eight passes in registers (fp32 rows of up to 2048, 16-bit rows of up to 4096): the same kernel with more
      // vectors per lane, every load of the row, the gain and the bias in flight at once
      if (L <= 6 * perWave) { LNL(6); return true; }
      LNL(8); return true;
#undef LNL
    }
    if (L <= perWave) { LN(64, 1, gw); return true; }
    if (L <= 2 * perWave) { LN(64, 2, gw); return true; }
    if (L <= 4 * perWave) { LN(64, 4, gw); return true; }
    if (L <= 8 * perWave) { LN(64, 8, gw); return true; }
    if (L <= 4 * perBlock) { LN(256, 4, gb); return true; }
    if (L <= 8 * perBlock) { LN(256, 8, gb); return true; }
#undef LN
    if (p.outerX.rank <= 1 && p.outerZ.rank <= 1 && L % V == 0 && p.rows < (1LL << 31)) {
      const LongType xp = p.outerX.rank ? p.outerX.stride[0] : 0, zp = p.outerZ.rank ? p.outerZ.stride[0] : 0;
      if (bt) hipLaunchKernelGGL((layernorm_long<T, true>), dim3((unsigned)p.rows), dim3(1024), 0, s, xt, gt, bt, zt, L, xp, zp, eps);
      else hipLaunchKernelGGL((layernorm_long<T, false>), dim3((unsigned)p.rows), dim3(1024), 0, s, xt, gt, bt, zt, L, xp, zp, eps);
      return true;
    }
  }
  if constexpr (sizeof(T) <= 4) {
    if (!vec && p.xInner == 1 && p.zInner == 1 && p.outerX.rank <= 1 && p.outerZ.rank <= 1 && L >= V && L / V <= 64 * 8 && L < (1 << 30)) {
      const LongType xp = p.outerX.rank ? p.outerX.stride[0] : 0, zp = p.outerZ.rank ? p.outerZ.stride[0] : 0;
      const LongType per = (L / V + 63) / 64;
      const bool nts = (size_t)p.rows * (size_t)L * sizeof(T) >= ((size_t)8 << 20);
#define LWR_(NV, B, NTS) hipLaunchKernelGGL((layernorm_wave_regs<T, NV, B, NTS>), dim3(gw), dim3(256), 0, s, xt, gt, bt, zt, p.rows, (int)L, xp, zp, eps)
#define LWR(NV) do { if (bt) { if (nts) LWR_(NV, true, true); else LWR_(NV, true, false); } else { if (nts) LWR_(NV, false, true); else LWR_(NV, false, false); } } while (0)
      if (per <= 1) LWR(1); else if (per <= 2) LWR(2); else if (per <= 4) LWR(4); else LWR(8);
#undef LWR
#undef LWR_
      return true;
    }
  }
  if (L <= 64 * 16) { hipLaunchKernelGGL((layernorm_rows<T, 64, 16, 1>), dim3(gw), dim3(256), 0, s, a, xt, gt, bt, zt, eps); return true; }
  if (L <= 256 * 32) { hipLaunchKernelGGL((layernorm_rows<T, 256, 32, 1>), dim3(gb), dim3(256), 0, s, a, xt, gt, bt, zt, eps); return true; }
  return false;   // longer rows: the caller takes the generic kernel
}

// x + addend -> sumOut, layer_norm(sumOut) -> z in one kernel; only the one-wave-per-row vector case (rows at a constant
// pitch, 16-byte aligned), anything else returns false and the caller runs the two ops
template <typename T>
static bool addLayerNormTyped(hipStream_t s, const void* x, const void* addend, void* sumOut, const void* gain, const void* bias, void* z, LongType rows,
                              LongType L, LongType xPitch, LongType aPitch, LongType sPitch, LongType zPitch, float eps) {
  constexpr int V = 16 / sizeof(T);
  auto al = [](const void* q) { return (reinterpret_cast<uintptr_t>(q) & 15) == 0; };
  if (L % V != 0 || L > 4 * 64 * V || L < V || !bias) return false;
  if (!al(x) || !al(addend) || !al(sumOut) || !al(gain) || !al(bias) || !al(z)) return false;
  if (xPitch % V || aPitch % V || sPitch % V || zPitch % V) return false;
  const unsigned gw = (unsigned)((rows + 3) / 4);
  const LongType perWave = 64 * V;
#define ALN(NV) hipLaunchKernelGGL((layernorm_linear<T, NV, true, 1, true>), dim3(gw), dim3(256), 0, s, (const T*)x, (const T*)gain, (const T*)bias, (T*)z, rows, (int)L, \
                                   xPitch, zPitch, eps, (const T*)addend, aPitch, (T*)sumOut, sPitch)
  if (L <= perWave) ALN(1);
  else if (L <= 2 * perWave) ALN(2);
  else if (L <= 3 * perWave) ALN(3);
  else ALN(4);
#undef ALN
  return true;
}
bool launchAddLayerNormRows(hipStream_t s, DataType dt, const void* x, const void* addend, void* sumOut, const void* gain, const void* bias, void* z,
                            LongType rows, LongType L, LongType xPitch, LongType aPitch, LongType sPitch, LongType zPitch, float eps) {
  if (rows == 0 || L == 0) return true;
  bool ok = false;
  switch (dt) {
    case FLOAT32: ok = addLayerNormTyped<float>(s, x, addend, sumOut, gain, bias, z, rows, L, xPitch, aPitch, sPitch, zPitch, eps); break;
    case HALF: ok = addLayerNormTyped<f16_t>(s, x, addend, sumOut, gain, bias, z, rows, L, xPitch, aPitch, sPitch, zPitch, eps); break;
    case BFLOAT16: ok = addLayerNormTyped<bf16_t>(s, x, addend, sumOut, gain, bias, z, rows, L, xPitch, aPitch, sPitch, zPitch, eps); break;
    default: ok = false;
  }
  if (ok) HIP_CHECK(hipGetLastError());
  return ok;
}

bool launchLayerNormRows(hipStream_t s, DataType dt, const void* x, const void* gain, const void* bias, void* z,
                         const RowPlan& p, float eps) {
  if (p.rows == 0 || p.rowLen == 0) return true;
  bool done = false;
  switch (dt) {
    case FLOAT32: done = layerNormTyped<float>(s, x, gain, bias, z, p, eps); break;
    case DOUBLE: done = layerNormTyped<double>(s, x, gain, bias, z, p, eps); break;
    case HALF: done = layerNormTyped<f16_t>(s, x, gain, bias, z, p, eps); break;
    case BFLOAT16: done = layerNormTyped<bf16_t>(s, x, gain, bias, z, p, eps); break;
    default: ND4J_THROW("layer_norm: unsupported dtype");
  }
  HIP_CHECK(hipGetLastError());
  return done;
}

// generic axes: one block per statistics group, elements reached through the inner walk; gain/bias are
// indexed by the coordinate along the channel axis
struct LnArgs {
  DevShape outerX, innerX, outerZ, innerZ;
  LongType outerLen, innerLen;
  int channelInInner, channelPos;
};
__device__ __forceinline__ LongType coordAt(const DevShape& s, LongType idx, int pos) {
  for (int d = s.rank - 1; d >= 0; d--) {
    LongType q = idx / s.shape[d], c = idx - q * s.shape[d];
    if (d == pos) return c;
    idx = q;
  }
  return 0;
}
template <typename T>
__global__ __launch_bounds__(256) void layernorm_generic(LnArgs a, const T* __restrict__ x, const T* __restrict__ gain,
                                                         const T* __restrict__ bias, T* __restrict__ z, float eps) {
  using A = typename Conv<T>::acc;
  __shared__ A lds[4];
  const LongType o = blockIdx.x;
  const LongType xb = walk<LongType>(a.outerX, o), zb = walk<LongType>(a.outerZ, o);
  A sum = (A)0;
  for (LongType j = threadIdx.x; j < a.innerLen; j += 256) sum += (A)to_float(x[xb + walk<LongType>(a.innerX, j)]);
  sum = block_allreduce<SumOp, 4, A>(sum, lds);
  const A mean = sum / (A)a.innerLen;
  A sq = (A)0;
  for (LongType j = threadIdx.x; j < a.innerLen; j += 256) { A d = (A)to_float(x[xb + walk<LongType>(a.innerX, j)]) - mean; sq += d * d; }
  sq = block_allreduce<SumOp, 4, A>(sq, lds);
  const A var = a.innerLen > 1 ? sq / (A)a.innerLen : (A)0;
  const A sd = r_sqrt<A>(var + (A)eps);
  const LongType cOuter = a.channelInInner ? 0 : coordAt(a.outerX, o, a.channelPos);
  for (LongType j = threadIdx.x; j < a.innerLen; j += 256) {
    const LongType c = a.channelInInner ? coordAt(a.innerX, j, a.channelPos) : cOuter;
    A y = ((A)to_float(x[xb + walk<LongType>(a.innerX, j)]) - mean) / sd;
    if (gain) y *= (A)to_float(gain[c]);   // no gain: the stand-alone standardize op
    if (bias) y += (A)to_float(bias[c]);
    z[zb + walk<LongType>(a.innerZ, j)] = Conv<T>::from(y);
  }
}
void launchLayerNormGeneric(hipStream_t s, DataType dt, const void* x, const void* gain, const void* bias, void* z,
                            const LnGenericPlan& p, float eps) {
  if (p.outerLen == 0 || p.innerLen == 0) return;
  ND4J_REQUIRE(p.outerLen < (1LL << 31), "layer_norm: too many groups");
  LnArgs a;
  a.outerX = p.outerX; a.innerX = p.innerX; a.outerZ = p.outerZ; a.innerZ = p.innerZ;
  a.outerLen = p.outerLen; a.innerLen = p.innerLen; a.channelInInner = p.channelInInner; a.channelPos = p.channelPos;
  dim3 g((unsigned)p.outerLen), b(256);
  switch (dt) {
    case FLOAT32: hipLaunchKernelGGL((layernorm_generic<float>), g, b, 0, s, a, (const float*)x, (const float*)gain, (const float*)bias, (float*)z, eps); break;
    case DOUBLE: hipLaunchKernelGGL((layernorm_generic<double>), g, b, 0, s, a, (const double*)x, (const double*)gain, (const double*)bias, (double*)z, eps); break;
    case HALF: hipLaunchKernelGGL((layernorm_generic<f16_t>), g, b, 0, s, a, (const f16_t*)x, (const f16_t*)gain, (const f16_t*)bias, (f16_t*)z, eps); break;
    case BFLOAT16: hipLaunchKernelGGL((layernorm_generic<bf16_t>), g, b, 0, s, a, (const bf16_t*)x, (const bf16_t*)gain, (const bf16_t*)bias, (bf16_t*)z, eps); break;
    default: ND4J_THROW("layer_norm: unsupported dtype");
  }
  HIP_CHECK(hipGetLastError());
}

}  // namespace nd4jhip
