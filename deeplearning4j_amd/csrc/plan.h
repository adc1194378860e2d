// Host-side planning: turns shapeInfo descriptors into the collapsed iteration records the kernels take.
#pragma once
#include <vector>

#include "kernels.h"
#include "runtime.h"

namespace nd4jhip {

// operands[0] is the output; all operands must have equal length
EwPlan buildEwPlan(const std::vector<const LongType*>& operands);

// dims: the dimensions to reduce (already normalised to [0, rank)); empty = reduce everything.
// zShapeInfo may carry unit dims (keepDims) which are skipped when lining z up with the kept dims.
ReducePlan buildReducePlan(const LongType* xShapeInfo, const LongType* zShapeInfo, const std::vector<LongType>& dims,
                           bool zLinear);

// rows along `dim` of x, written along `dim` of z
RowPlan buildRowPlan(const LongType* xShapeInfo, const LongType* zShapeInfo, int dim);

// collapse a (shape, strides...) set: drops unit dims and merges neighbours that are jointly dense.
// strides[o] are per-operand stride arrays of length rank; returns the new rank.
int collapseDims(int rank, LongType* shape, LongType* const* strides, int nOperands);

DevShape toDevShape(const std::vector<LongType>& shape, const std::vector<LongType>& stride);

std::vector<LongType> normalizeDims(int rank, const LongType* dims, LongType n, const char* what);

}  // namespace nd4jhip
