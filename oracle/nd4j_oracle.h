/*
 * CPU oracle for the libnd4j data-parallel op path -- TEST INFRASTRUCTURE ONLY.
 *
 * A plain-C restatement of the reference's CPU algorithms, written from the
 * reference sources cited on every function.  Only tests/, the smoke check and
 * the benchmark's cpu_baseline leg may link or load this library; the product
 * library never calls into it.
 *
 * Conventions
 *   - every array is (buffer pointer, shapeInfo pointer); buffer already points
 *     at the first element of the view (offset applied once by the caller)
 *   - shapeInfo is the reference descriptor int64[2*rank+4]:
 *       [rank, shape.., stride.., extra(flags|dtype bits), ews, order]
 *     (libnd4j/include/helpers/shape.h:76-104)
 *   - dtype codes follow libnd4j/include/array/DataType.h:26-50
 *   - fp16/bf16 arrays: values are widened to float, the op is evaluated in
 *     float, the result is rounded once (RNE).  The reference's literal half
 *     arithmetic (re-rounding after every scalar step) is offered only where a
 *     function has a `literal_half` switch, to report its deviation.
 *   - return value 0 = ok, non-zero = unsupported argument combination
 *
 * Pinning status (what checks each function besides this restatement):
 *   shape/offset walk, TAD ............ brute force vs numpy strided views
 *   hash .............................. reference vectors HashUtilsTests.cpp:28-41
 *   pairwise .......................... NativeOpsTests.cpp:170-186, bit-exact vs numpy
 *   transform strict/float ............ NativeOpsTests.cpp:658-760, closed forms
 *                                       TestTransformOpValidation.java:1043-1054
 *   transform strict, rest of table ... library routines (numpy/scipy), identities, and central
 *   (tests/test_oracle_tail_ops.py)     differences of the primal op for every *Derivative op;
 *                                       PreciseGELUDerivative away from zero: parity unpinned (the
 *                                       reference cubes the scaled argument; only f'(x)+f'(-x)=1 and the
 *                                       values near zero are pinned)
 *   transform same, pairwise/scalar/
 *   broadcast tables, rest of tables .. numpy / math routines per function, table numbering per opNum,
 *                                       broadcast vs numpy broadcasting over TADs
 *   reduce same/float ................. NativeOpsTests.cpp:209-238, fp64 bounds; entropies vs scipy.stats
 *   reduce3 ........................... NDArrayTests.cpp:1455-1488, NDArrayTests2.cpp:1144-1152 (Euclidean), scipy.spatial
 *   summary stats, counts, Any/All,
 *   transform bool .................... numpy var/std (ddof 0/1), count_nonzero, isnan/isinf/isfinite
 *   index reduce / argmax ............. NativeOpsTests.cpp:84-117, LegacyOpsTests.cpp:279-310,
 *                                       DeclarableOpsTests1.cpp:2197-2300, brute force
 *   top_k ............................. DeclarableOpsTests5.cpp:1074-1245 (Test_TopK_0..5), brute force
 *                                       on tie-free rows; behaviour on repeated values: source only
 *   shape ops (oracle.py, numpy) ...... strided_slice: IndexingTests.cpp:34-330, DeclarableOpsTests4.cpp:1268-1336,
 *                                       DeclarableOpsTests6.cpp:40-215 (tests/golden/strided_slice_vectors.json) and
 *                                       brute force over python ranges; negative steps and reshape order 'f':
 *                                       parity unpinned (numpy semantics only)
 *   gradient ops (oracle.py, numpy) ... softmax_bp, standardize_bp, layer_norm_bp, matmul_bp: central differences of the
 *                                       pinned forward restatements (tests/test_oracle_bp_ops.py); the reference's own
 *                                       tests hold shapes and all-zero cases only (DeclarableOpsTests15.cpp:72-90,397-408,484-512)
 *   xw_plus_b ......................... composition of matmul and the bias row (xw_plus_b.cpp:117-133)
 *   matmul ............................ DeclarableOpsTests14.cpp:601-1260, DeclarableOpsTests19.cpp:52-140
 *   softmax ........................... DeclarableOpsTests1.cpp:2523-2740; inf/nan clamp
 *                                       semantics: parity unpinned (source only)
 *   clip_by_value, affine, scaled_tanh,
 *   stabilize, set_range
 *   (oracle.py, numpy) ................ DeclarableOpsTests1.cpp:801-848 (ClipByValue1/2), numpy.clip, library tanh; stabilize and
 *                                       set_range: hand-computed cases and invariants only (the reference has no test of them)
 *   log_softmax (oracle.py, numpy) .... DeclarableOpsTests5.cpp:2199-2340 (tests/golden/log_softmax_vectors.json)
 *   layer_norm ........................ closed form (TestLayerOpValidation.java:1188-1333)
 *   dot_product_attention_v2 .......... parity unpinned: the reference has no enabled
 *                                       test; pinned only as matmul+softmax composition
 *                                       and a textbook causal mask; query / value masks: the padded-batch identity
 *                                       (masked keys == truncated keys) and the manual composition of
 *                                       TestReductionOpValidation.java:1291-1327 (tests/test_oracle_attention_masks.py)
 *   match-condition ops, norm_p,
 *   equals_with_eps (oracle.py, numpy)  NDArrayTests2.cpp:96-103 (FirstIndex), BooleanIndexingTest.java:208-335
 *                                       (CompareAndSet / CompareAndReplace / MatchCondition cases), closed forms
 *                                       (tests/test_oracle_cond_ops.py)
 *   remaining pairwise / scalar ops
 *   (oracle.py, numpy) ................ igamma / igammac: DeclarableOpsTests10.cpp:481-515 and scipy.special.gammainc (exact for
 *                                       x < 1, within the truncation of the reference's series beyond); relative errors, axpy,
 *                                       pow_derivative, log_poisson_loss: closed forms, central differences, Stirling's bound
 *                                       (tests/test_oracle_pairwise_params.py)
 *   integer arrays .................... no restatement: the GPU tests compare with numpy's integer arithmetic directly
 */
#ifndef ND4J_ORACLE_H
#define ND4J_ORACLE_H
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { ORC_BOOL = 1, ORC_HALF = 3, ORC_FLOAT32 = 5, ORC_DOUBLE = 6, ORC_INT32 = 9, ORC_INT64 = 10, ORC_BFLOAT16 = 17 };

/* descriptor helpers */
int64_t orc_shape_info_length(int rank);
void orc_make_shape_info(int rank, const int64_t *shape, const int64_t *strides /*NULL = dense in `order`*/, int dtype,
                         char order, int64_t *out);
int64_t orc_length(const int64_t *si);
int orc_dtype(const int64_t *si);
int64_t orc_offset(const int64_t *si, int64_t linearIndex);

/* half conversions */
uint16_t orc_f32_to_bf16(float f);
float orc_bf16_to_f32(uint16_t h);
uint16_t orc_f32_to_f16(float f);
float orc_f16_to_f32(uint16_t h);

/* op-name hash */
int64_t orc_hash(const char *name);

/* TAD pack: returns number of TADs; tadShapeInfo must hold 2*rank+4 entries, offsets numTads entries (or NULL) */
int64_t orc_tad(const int64_t *si, const int64_t *dims, int ndims, int64_t *tadShapeInfo, int64_t *offsets);

/* legacy loops */
int orc_pairwise(int opNum, const void *x, const int64_t *xsi, const void *y, const int64_t *ysi, void *z,
                 const int64_t *zsi);
int orc_transform_strict(int opNum, const void *x, const int64_t *xsi, void *z, const int64_t *zsi);
int orc_transform_float(int opNum, const void *x, const int64_t *xsi, void *z, const int64_t *zsi);
int orc_transform_same(int opNum, const void *x, const int64_t *xsi, void *z, const int64_t *zsi);
int orc_transform_bool(int opNum, const void *x, const int64_t *xsi, void *z, const int64_t *zsi);
int orc_summary_stats(int opNum, const void *x, const int64_t *xsi, void *z, const int64_t *zsi, const int64_t *dims, int ndims,
                      int biasCorrected);
int orc_reduce3(int opNum, const void *x, const int64_t *xsi, const void *y, const int64_t *ysi, void *z, const int64_t *zsi,
                const int64_t *dims, int ndims);
int orc_reduce_count(int kind, const void *x, const int64_t *xsi, void *z, const int64_t *zsi, const int64_t *dims, int ndims);
int orc_scalar(int opNum, const void *x, const int64_t *xsi, double scalar, void *z, const int64_t *zsi);
int orc_broadcast(int opNum, const void *x, const int64_t *xsi, const void *y, const int64_t *ysi, void *z,
                  const int64_t *zsi, const int64_t *dims, int ndims);
int orc_reduce_same(int opNum, const void *x, const int64_t *xsi, void *z, const int64_t *zsi, const int64_t *dims,
                    int ndims);
int orc_reduce_float(int opNum, const void *x, const int64_t *xsi, void *z, const int64_t *zsi, const int64_t *dims,
                     int ndims);
int orc_index_reduce(int opNum, const void *x, const int64_t *xsi, void *z, const int64_t *zsi, const int64_t *dims,
                     int ndims);

/* declarable ops */
int orc_top_k(const void *x, const int64_t *xsi, void *values, const int64_t *vsi, void *indices, const int64_t *isi,
              int64_t k, int needSort);
int orc_softmax(const void *x, const int64_t *xsi, void *z, const int64_t *zsi, int dim, int literal_half);
int orc_layer_norm(const void *x, const int64_t *xsi, const void *gain, const int64_t *gsi, const void *bias,
                   const int64_t *bsi, void *z, const int64_t *zsi, const int64_t *axes, int naxes, int channelsFirst);
/* accumulate: 0 = sequential k-loop in the output dtype (usualGemm), 1 = float accumulator, 2 = double accumulator */
int orc_matmul(const void *x, const int64_t *xsi, const void *y, const int64_t *ysi, void *z, const int64_t *zsi,
               int transX, int transY, int transZ, double alpha, double beta, int accumulate);
int orc_attention_v2(const void *q, const int64_t *qsi, const void *v, const int64_t *vsi, const void *k,
                     const int64_t *ksi, void *out, const int64_t *osi, void *weights, const int64_t *wsi,
                     void *logits, const int64_t *lsi, double scale, int causal, const void *qmask,
                     const int64_t *qmsi, const void *vmask, const int64_t *vmsi);

/* decoder glue (broadcast add of a row vector, gather of rows) used by the decode harness check */
int orc_add_row_vector(const void *x, const int64_t *xsi, const void *row, const int64_t *rsi, void *z,
                       const int64_t *zsi);

void orc_set_threads(int n);
int orc_get_threads(void);

#ifdef __cplusplus
}
#endif
#endif
