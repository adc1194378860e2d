// Host-callable launchers of the HIP kernels.  Callers (the facade) validate dtypes and shapes and
// build the plans; launchers only pick a kernel variant and a grid.
#pragma once
#include <hip/hip_runtime.h>

#include "types.h"

namespace nd4jhip {

// ---- elementwise ---------------------------------------------------------------------------------
enum UnaryKind : int {
  // TransformStrict (loops/legacy_ops.h:54-64 of the reference)
  U_COS, U_EXP, U_LOG, U_SIGMOID, U_SIN, U_SOFTPLUS, U_TANH, U_SWISH, U_ERF, U_GELU, U_PRECISE_GELU,
  // TransformFloat (legacy_ops.h:67)
  U_SQRT, U_RSQRT,
  // TransformSame (legacy_ops.h:40-44) and TransformAny Assign (legacy_ops.h:46)
  U_ABS, U_NEG, U_SQUARE, U_RECIPROCAL, U_IDENTITY, U_ONE_MINUS, U_CUBE,
  U_COUNT,
  // The rest of the transform tables: one kernel per dtype with the op chosen at run time (U_TAIL_FIRST ..).
  // TransformStrict
  U_TAIL_FIRST = 64,
  U_TANH_D = U_TAIL_FIRST, U_SIGMOID_D, U_SOFTSIGN_D, U_TAN_D, U_SELU_D, U_RATIONAL_TANH_D, U_RECTIFIED_TANH_D, U_SWISH_D,
  U_ACOSH_D, U_ASINH_D, U_SINH_D, U_LOG_SIGMOID_D, U_SPECIAL_D, U_CUBE_D, U_ACOS, U_ASIN, U_ATAN, U_HARD_TANH,
  U_SOFTSIGN, U_HARD_SIGMOID, U_RATIONAL_TANH, U_RECTIFIED_TANH, U_SINH, U_COSH, U_TAN, U_SELU, U_LOG1P, U_ACOSH,
  U_ASINH, U_RINT, U_LOG_SIGMOID, U_ERFC, U_EXPM1, U_ATANH, U_GELU_D, U_PRECISE_GELU_D, U_MISH, U_MISH_D,
  // TransformSame
  U_ONES, U_ROUND, U_TIMES_ONE_MINUS, U_CEIL, U_FLOOR,
  U_SIGN_REF,         // TransformSame Sign as the reference's macro evaluates it: 1 for every non-zero number, -1 for zero and NaN
  U_STABILIZE_FP16,   // TransformStrict StabilizeFP16: 2^-14 (the smallest normal HALF) for x <= 0, else x
  // TransformBool (output type BOOL)
  U_IS_INF, U_IS_NAN, U_IS_FINITE, U_IS_INF_OR_NAN, U_IS_POSITIVE, U_NOT, U_IS_NEGATIVE,
  U_TAIL_END
};
enum PairwiseKind : int {
  P_ADD, P_COPY, P_DIV, P_MUL, P_RSUB, P_SUB, P_MAX, P_MIN, P_RDIV, P_SQSUB, P_COUNT,
  // The rest of the pairwise / scalar / broadcast tables, op chosen at run time (P_TAIL_FIRST ..)
  P_TAIL_FIRST = 64,
  P_POW = P_TAIL_FIRST, P_REMAINDER, P_FMOD, P_ATAN2, P_TRUNCATE_DIV, P_FLOOR_DIV, P_FLOOR_MOD, P_REVERSE_MOD,
  P_SAFE_DIVIDE, P_MOD, P_LOGICAL_OR, P_LOGICAL_XOR, P_LOGICAL_NOT, P_LOGICAL_AND, P_AMAX, P_AMIN, P_TRUNCATE_MOD,
  P_REPLACE_NANS, P_DIVIDE_NO_NAN,
  // scalar table only
  P_ELU, P_ELU_D, P_LEAKY_RELU, P_LEAKY_RELU_D, P_LOG_X, P_RELU, P_RELU6, P_RELU_D, P_STEP, P_LSTM_CLIP,
  P_SQ_RSUB, P_REVERSE_POW, P_SXE_LOGITS_SMOOTHER,
  // pairwise / scalar ops that need no parameter although the executioner may pass some
  P_REL_ERR, P_POW_DERIV, P_LOG_POISSON, P_LOG_POISSON_FULL, P_IGAMMA, P_IGAMMAC,
  // comparisons (the bool tables): 1 / 0, stored into a BOOL output
  P_EQ, P_NE, P_GT, P_GE, P_LT, P_LE,
  P_TAIL_END
};

// Joint iteration plan of up to three operands of equal length.
struct EwPlan {
  int nOperands = 0;       // operand 0 is the output
  LongType length = 0;
  bool sameShape = true;   // false: every operand is walked through its own shape (own[])
  bool contiguous = false; // collapsed rank 1 and unit strides everywhere
  bool index32 = true;     // length and every reachable offset fit 31 bits
  int rank = 0;            // collapsed common shape
  LongType shape[MAX_DEV_RANK];
  LongType stride[3][MAX_DEV_RANK];
  DevShape own[3];
};

void launchUnary(hipStream_t s, UnaryKind k, DataType xdt, DataType zdt, const void* x, void* z, const EwPlan& p);
void launchPairwise(hipStream_t s, PairwiseKind k, DataType xdt, DataType ydt, DataType zdt, const void* x,
                    const void* y, void* z, const EwPlan& p);
// z = f(x; s1, s2): the transforms of the legacy tables that read two extra parameters
enum Scalar2Kind : int {
  S2_CLIP_BY_VALUE,   // x > s2 ? s2 : (x < s1 ? s1 : x)      ops.h:412-415, helpers/cpu/clip.cpp:211-219
  S2_AFFINE,          // s1 * x + s2                          ops.h:453
  S2_SCALED_TANH,     // s1 * tanh(s2 * x)                    ops.h:1088-1090
  S2_STABILIZE,       // x * s1 beyond +-3.79297773665: that cutoff / s1, else x   ops.h:458-468 (one parameter)
  S2_SET_RANGE        // x inside [s1, s2]: x; else floor(v * (s2 - s1)) + s1 with v = sigmoid(x) for the range [0, 1], else x   ops.h:427-438
};
void launchScalar2Op(hipStream_t s, Scalar2Kind k, DataType xdt, DataType zdt, const void* x, double s1, double s2, void* z,
                     const EwPlan& p);
// z = x (op) scalar
void launchScalarOp(hipStream_t s, PairwiseKind k, DataType dt, const void* x, double scalar, void* z, const EwPlan& p);

// Integer / bool arrays (intops.hip).  launchUnary, launchPairwise, launchScalarOp, launchReduce and launchIndexReduce
// route there by themselves when every operand is of an integer type; these are the direct entry points.
bool isIntLike(DataType t);
// k is a UnaryKind (binary false) or a PairwiseKind (binary true; y, or `scalar` when hasScalar)
void launchIntElementwise(hipStream_t s, int k, bool binary, DataType xdt, DataType ydt, DataType zdt, const void* x, const void* y,
                          void* z, const EwPlan& p, LongType scalar, bool hasScalar);

// Ops that test a "match condition" read from the extra parameters (condops.hip)
enum CondKind : int {
  C_MATCH_BOOL, C_SET_TRANSFORM, C_SET, C_REPLACE, C_AXPY, C_BIN_REL_ERR, C_BIN_MIN_ABS_REL_ERR,
  // the members of the bool tables that are not plain comparisons (ops.h:1051-1063, 1755-1790, 1896-1925): compare holds the
  // one extra parameter, mode whether the caller passed any
  C_BOOL_EPSILON, C_BOOL_AND, C_BOOL_OR, C_BOOL_XOR
};
enum CondReduceKind : int { CR_COUNT, CR_FIRST, CR_LAST };
struct CondParams {
  int mode = 0;
  double compare = 0, set = 0, eps = 0;   // as the array's type holds them
  int xdt = FLOAT32;                      // the type the comparisons run in
};
void launchCondElementwise(hipStream_t s, CondKind kind, const CondParams& c, DataType ydt, DataType zdt, const void* x, const void* y,
                           void* z, const EwPlan& p, double scalar, bool hasScalar);

// ---- reductions ----------------------------------------------------------------------------------
enum ReduceKind : int {
  R_SUM, R_MAX, R_MIN, R_PROD, R_ASUM, R_AMAX, R_AMIN,        // ReduceSame 0..6
  R_MEAN, R_AMEAN, R_NORM1, R_NORM2, R_NORMMAX, R_SQNORM,     // ReduceFloat 0,1,2,3,4,7
  R_ENTROPY, R_LOG_ENTROPY, R_SHANNON_ENTROPY,               // ReduceFloat 8,9,10
  R_COUNT
};
enum IndexKind : int { I_MAX, I_MIN, I_AMAX, I_AMIN, I_COUNT };
// reductions whose accumulator or output type differs from the input's: summary statistics (double triple n, mean, M2),
// counts (INT64 out), Any / All (BOOL out)
enum MiscReduceKind : int {
  M_VARIANCE, M_STDDEV, M_COUNT_NONZERO, M_COUNT_ZERO, M_ANY, M_ALL,
  // two-operand reductions (reduce3), z in a float type
  M3_MANHATTAN, M3_EUCLIDEAN, M3_COSINE_SIMILARITY, M3_DOT, M3_COSINE_DISTANCE, M3_JACCARD, M3_HAMMING,
  M3_EQUALS_EPS,   // 1 when |x - y| <= param everywhere, else 0 (Reduce3 EqualsWithEps)
  M_NORMP,         // (sum |x|^param)^(1 / param), z in a float type (ReduceFloat NormP); not a two-operand kind
  // ReduceBool 2-7: 1 when any element is finite / inf or nan / nan / inf / positive / negative (sum of indicators, ops.h:1139-1163)
  M_ANY_FINITE, M_ANY_INF_OR_NAN, M_ANY_NAN, M_ANY_INF, M_ANY_POSITIVE, M_ANY_NEGATIVE,
  // the ReduceFloat table for an input type that differs from the output's (any numeric X into any float Z); the
  // ReduceKind travels in `param`
  M_REDUCE_FLOAT
};

// outer = kept dims (one output element each), inner = reduced dims
struct ReducePlan {
  DevShape outer;        // strides into x
  DevShape inner;        // strides into x
  DevShape zOuter;       // same shape as outer, strides into z
  LongType outerLen = 1, innerLen = 1;
  bool index32 = true;
  bool zLinear = false;  // write z[o] instead of walking zOuter (index reduce)
};

void launchReduce(hipStream_t s, ReduceKind k, DataType xdt, DataType zdt, const void* x, void* z, const ReducePlan& p,
                  void* scratch, size_t scratchBytes);
// Full reduction of a dense vector x[n] into z[1] whose cross-block partials live in a fixed device array instead of
// allocated scratch: no allocation on any path.  reduceNoAllocScratch() resolves that array's address on the current
// device (once per device); same kernels and split rule as launchReduce, hence the same bits.
constexpr size_t NOALLOC_SCRATCH_BYTES = 64 * 1024;
constexpr LongType NOALLOC_MAX_ELEMENTS = (1LL << 31) - 1;
void* reduceNoAllocScratch();
void launchReduceScalarNoAlloc(hipStream_t s, ReduceKind k, DataType dt, const void* x, LongType n, void* z);
// zdt: the float type for variance / standard deviation, INT64 for counts, BOOL for Any / All
void launchReduceMisc(hipStream_t s, MiscReduceKind k, DataType xdt, DataType zdt, const void* x, void* z, const ReducePlan& p,
                      bool biasCorrected, void* scratch, size_t scratchBytes, const void* y = nullptr, DataType ydt = FLOAT32,
                      const ReducePlan* yPlan = nullptr, double param = 0.0);
// count of elements that meet the condition / position of the first or last one (-1: none); z INT32 or INT64
struct ReducePlan;
void launchCondReduce(hipStream_t s, CondReduceKind kind, const CondParams& c, DataType zdt, const void* x, void* z, const ReducePlan& p,
                      void* scratch, size_t scratchBytes);
void launchIndexReduce(hipStream_t s, IndexKind k, DataType xdt, DataType zdt, const void* x, void* z,
                       const ReducePlan& p, void* scratch, size_t scratchBytes);

// kind: a ReduceKind of the ReduceSame table (isIndex false) or an IndexKind (isIndex true)
void launchIntReduce(hipStream_t s, int kind, bool isIndex, DataType xdt, DataType zdt, const void* x, void* z, const ReducePlan& p,
                     void* scratch, size_t scratchBytes);

// ---- row ops ---------------------------------------------------------------------------------------
struct RowPlan {
  DevShape outerX;     // row start offsets of the input
  DevShape outerZ;     // row start offsets of the output
  LongType rows = 1, rowLen = 1;
  LongType xInner = 1, zInner = 1;  // element stride along the row
  bool index32 = true;
};
// clampMode: true = the reference's same-shape branch (finite max, +-88 clamp, sum floor 1e-6)
void launchSoftmax(hipStream_t s, DataType dt, const void* x, void* z, const RowPlan& p, bool clampMode);
// log(exp(x - max) / sum) along the plan's rows, evaluated in that order
void launchLogSoftmax(hipStream_t s, DataType dt, const void* x, void* z, const RowPlan& p);
// false: the rows are longer than the row kernels take (nothing launched; launchLayerNormGeneric serves them)
bool launchLayerNormRows(hipStream_t s, DataType dt, const void* x, const void* gain, const void* bias, void* z,
                         const RowPlan& p, float eps);
// sumOut = x + addend (pairwise Add in the array type), z = layer_norm(sumOut) over rows of length L at constant pitches, in
// one kernel; false when the shape is not the one-wave-per-row vector case (nothing launched then)
bool launchAddLayerNormRows(hipStream_t s, DataType dt, const void* x, const void* addend, void* sumOut, const void* gain, const void* bias,
                            void* z, LongType rows, LongType L, LongType xPitch, LongType aPitch, LongType sPitch, LongType zPitch, float eps);
// gradI = softmaxed * (gradO - sum_row(softmaxed * gradO)); pg = row plan (gradO, gradI), ps = (softmaxed, gradI)
void launchSoftmaxBp(hipStream_t s, DataType dt, const void* gradO, const void* softmaxed, void* gradI, const RowPlan& pg,
                     const RowPlan& ps);
// k largest elements of every row (last axis) with their positions; pv / pi are the row plans (x, values) and
// (x, indices); sorted: descending values, else ascending positions
void launchTopK(hipStream_t s, DataType xdt, DataType idt, const void* x, void* values, void* indices, const RowPlan& pv,
                const RowPlan& pi, int k, bool sorted);
// generic layer norm over arbitrary axes: one block per statistics group
struct LnGenericPlan {
  DevShape outerX, innerX, outerZ, innerZ;
  LongType outerLen = 1, innerLen = 1;
  int channelInInner = 1;   // does the gain/bias axis belong to the reduced set
  int channelPos = 0;       // its position inside that set
};
void launchLayerNormGeneric(hipStream_t s, DataType dt, const void* x, const void* gain, const void* bias, void* z,
                            const LnGenericPlan& p, float eps);
// gradient of standardize over the plan's groups; gain (may be null) scales eps along the channel axis first.
// px walks (x, z), pe walks eps in its outerX / innerX members.
void launchStandardizeBp(hipStream_t s, DataType dt, const void* x, const void* eps, const void* gain, void* z,
                         const LnGenericPlan& px, const LnGenericPlan& pe);

// ---- GEMM ------------------------------------------------------------------------------------------
// Extra outputs a product can write from its epilogue, each what a separate op would have computed from the stored result
// C (same rounding points), so that a recorded op sequence "product, then an elementwise op on it" can run as one kernel:
//   act:   actOut[m][n] = GELU(C[m][n])                       (the legacy transform opNum 53 applied to C)
//   copy:  dst[m * dstRow + n - c0] = C[m][n] for c0 <= n < c1   (an assign of a column slice of C, e.g. into a key / value cache)
//   res:   resOut[m][n] = resIn[m][n] + C[m][n]               (a pairwise Add of C to another array of the same shape)
// Rows have unit column stride everywhere.  Only some kernels carry these (the decode-step ones); launchGemm says whether
// the one it chose did.
struct GemmEpilogue {
  int act = 0;              // 0 none, 1 GELU as the dense 16-bit transform evaluates it, 2 GELU in its full-precision form
  void* actOut = nullptr;
  LongType actRow = 0;
  int nCopy = 0;
  struct Copy { void* dst; LongType c0, c1, dstRow; } copy[2] = {{nullptr, 0, 0, 0}, {nullptr, 0, 0, 0}};
  const void* resIn = nullptr;
  void* resOut = nullptr;
  LongType resInRow = 0, resOutRow = 0;
};
struct GemmDesc {
  LongType M = 0, N = 0, K = 0, batch = 1;
  LongType aRow = 0, aCol = 0;   // element strides of op(A)[m][k]
  LongType bRow = 0, bCol = 0;   // element strides of op(B)[k][n]
  LongType cRow = 0, cCol = 0;
  LongType aBatch = 0, bBatch = 0, cBatch = 0;
  // optional second batch level: entry i of `batch` = (i / batchInner, i % batchInner), the outer index moving
  // by the *Batch2 strides (batchInner = 0: one level)
  LongType batchInner = 0, aBatch2 = 0, bBatch2 = 0, cBatch2 = 0;
  float alpha = 1.f, beta = 0.f;
  const void* bias = nullptr;   // optional dense [N] row (type of C) added to every output row
  const GemmEpilogue* epi = nullptr;
  // optional prologue: op(A) is one row (M = 1) or 5 to 32 rows, and what is multiplied is layer_norm(row; lnGain, lnBias,
  // lnEps) over each row's K elements, which also goes to lnOut (rows lnOutRow elements apart).  Counts as an epilogue
  // request for the return value of launchGemm: kernels that cannot do it launch nothing.
  const void* lnGain = nullptr;
  const void* lnBias = nullptr;
  void* lnOut = nullptr;
  LongType lnOutRow = 0;
  float lnEps = 1e-5f;
  // other optional prologue (one row, M = 1): op(A) is the output row of an attention whose key range was cut into attnSplits
  // parts -- the row is merged from the parts' records in attnPartial (heads of attnD values side by side along K) on the way in
  // and also written to attnOut, where the attention's own merge kernel would have put it.  Counts like the one above.
  const float* attnPartial = nullptr;
  int attnSplits = 0, attnD = 0;
  void* attnOut = nullptr;
};
// Returns true when every requested epilogue output was written; false: C was computed by a kernel without them and the
// caller runs the follow-up ops itself (always true without an epilogue request).
bool launchGemm(hipStream_t s, DataType dt, const void* A, const void* B, void* C, const GemmDesc& d);
// name of the kernel the calling thread's most recent launchGemm chose
const char* lastGemmKernel();

// ---- attention -------------------------------------------------------------------------------------
struct AttnDesc {
  LongType B = 0, Tq = 0, Tv = 0, D = 0, Dv = 0;   // B counts all batch entries (outer x H)
  LongType qB = 0, qT = 0, kB = 0, kT = 0, vB = 0, vT = 0, oB = 0, oT = 0;  // innermost stride is 1
  // optional second batch level (e.g. [batch, heads, T, D] views of token-major buffers): entry i of B is
  // (i / H, i % H); *B strides move the inner (head) index, *B2 the outer one.  H = 0: one level.
  LongType H = 0, qB2 = 0, kB2 = 0, vB2 = 0, oB2 = 0;
  float scale = 1.f;
  bool applyScale = false;
  bool causal = false;
  float maskValue = 1e9f;
  const unsigned char* vmask = nullptr;   // optional value (padding) mask, dense [B, Tv] bytes: 0 = masked key
  // decode kernel only: the keys of every (batch entry, query) cut into `splits` ranges, one block each, which leave
  // partial results in `partial` ([B * Tq][splits][ATTN_PART_PITCH(D)] floats); a merge kernel then writes `out` unless
  // mergeLater is set (the caller's next kernel merges on its way in)
  int splits = 1;
  float* partial = nullptr;
  bool mergeLater = false;
};
// how many key ranges the decode kernel should cut a problem into (1: do not cut)
int attentionDecodeSplits(const AttnDesc& d);
// fused path (no logits/weights written)
bool attentionFusedSupported(DataType dt, const AttnDesc& d);
// the host-made block order of the fused attention kernels (see BlockOrder in attention.hip): fills items, returns their number or 0
int attentionBlockOrder(int nBatch, int qTiles, int keyTilesPerQueryTile, int resident, unsigned short* items);
void launchAttentionFused(hipStream_t s, DataType dt, const void* q, const void* k, const void* v, void* out,
                          const AttnDesc& d);
// a few query rows against a long history, no causal mask (decode steps with a key/value cache)
bool attentionDecodeSupported(DataType dt, const AttnDesc& d);
// the merge step of a cut-up decode attention on its own (d.splits, d.partial as given to launchAttentionDecode with mergeLater)
void launchAttentionDecodeMerge(hipStream_t s, DataType dt, void* out, const AttnDesc& d);
void launchAttentionDecode(hipStream_t s, DataType dt, const void* q, const void* k, const void* v, void* out,
                           const AttnDesc& d);
// logits[b,i,j] = clip(scale * logits, +-1e4) - mask  (in place, row-major [B,Tq,Tv])
void launchAttentionLogitsFixup(hipStream_t s, DataType dt, void* logits, const AttnDesc& d);
// weights[b, i, :] *= qmask[b, i] (in place; qmask dense [B, Tq] of the weights' type)
void launchAttentionQueryMask(hipStream_t s, DataType dt, void* weights, const void* qmask, const AttnDesc& d);

// ---- misc ------------------------------------------------------------------------------------------
// z[i, :] = table[idx[i], :]
void launchGatherRows(hipStream_t s, DataType dt, DataType idxDt, const void* table, const void* idx, void* z,
                      LongType nIdx, LongType rowLen, LongType tableRows);
void launchFill(hipStream_t s, void* p, int byteValue, size_t bytes);

}  // namespace nd4jhip
