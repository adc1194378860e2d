// Basic types shared by host runtime and device kernels: dtype codes, the shapeInfo descriptor
// accessors and the fixed-rank device-side shape record that kernels take by value.
#pragma once
#include <cstdint>
#include <cstddef>

namespace nd4jhip {

typedef long long LongType;

// dtype codes, same numbering as the reference (libnd4j/include/array/DataType.h:26-50)
enum DataType : int {
  INHERIT = 0, BOOL = 1, FLOAT8 = 2, HALF = 3, HALF2 = 4, FLOAT32 = 5, DOUBLE = 6, INT8 = 7, INT16 = 8,
  INT32 = 9, INT64 = 10, UINT8 = 11, UINT16 = 12, UINT32 = 13, UINT64 = 14, QINT8 = 15, QINT16 = 16,
  BFLOAT16 = 17, UTF8 = 50, UTF16 = 51, UTF32 = 52, ANY = 100, AUTO = 200, UNKNOWN = 255
};

// flag bits of the descriptor's "extra" word (libnd4j/include/array/ArrayOptions.h:41-97)
constexpr LongType ARRAY_EMPTY = 8;
constexpr LongType ARRAY_BHALF = 2048;
constexpr LongType ARRAY_HALF = 4096;
constexpr LongType ARRAY_FLOAT = 8192;
constexpr LongType ARRAY_DOUBLE = 16384;
constexpr LongType ARRAY_CHAR = 32768;
constexpr LongType ARRAY_SHORT = 65536;
constexpr LongType ARRAY_INT = 131072;
constexpr LongType ARRAY_LONG = 262144;
constexpr LongType ARRAY_BOOL = 524288;
constexpr LongType ARRAY_UNSIGNED = 8388608;
constexpr LongType ARRAY_IS_VIEW = 33554432;
constexpr LongType ARRAY_ALL_DTYPE_BITS =
    ARRAY_BHALF | ARRAY_HALF | ARRAY_FLOAT | ARRAY_DOUBLE | ARRAY_CHAR | ARRAY_SHORT | ARRAY_INT | ARRAY_LONG |
    ARRAY_BOOL | ARRAY_UNSIGNED | 1048576 | 4194304 | 16777216;

constexpr int MAX_RANK = 32;     // what a descriptor may carry (reference SD_MAX_RANK)
constexpr int MAX_DEV_RANK = 8;  // what the kernels walk after dimension collapsing

inline size_t sizeOf(DataType t) {
  switch (t) {
    case BOOL: case INT8: case UINT8: case QINT8: case FLOAT8: return 1;
    case HALF: case BFLOAT16: case INT16: case UINT16: case QINT16: return 2;
    case FLOAT32: case INT32: case UINT32: case HALF2: return 4;
    case DOUBLE: case INT64: case UINT64: return 8;
    default: return 0;
  }
}
inline bool isFloatType(DataType t) { return t == HALF || t == BFLOAT16 || t == FLOAT32 || t == DOUBLE; }
inline const char* dtypeName(DataType t) {
  switch (t) {
    case BOOL: return "BOOL"; case HALF: return "HALF"; case FLOAT32: return "FLOAT"; case DOUBLE: return "DOUBLE";
    case INT8: return "INT8"; case INT16: return "INT16"; case INT32: return "INT32"; case INT64: return "INT64";
    case UINT8: return "UINT8"; case UINT16: return "UINT16"; case UINT32: return "UINT32"; case UINT64: return "UINT64";
    case BFLOAT16: return "BFLOAT16"; default: return "UNKNOWN";
  }
}

// --- shapeInfo accessors (libnd4j/include/helpers/shape.h:76-104,1804-1822) ------------------
// descriptor = [rank, shape.., stride.., extra, ews, order]; rank 0 has length 6 with extra at index 3.
namespace shape {
inline int rank(const LongType* si) { return (int)si[0]; }
inline int shapeInfoLength(int rank) { return rank == 0 ? 6 : 2 * rank + 4; }
inline const LongType* shapeOf(const LongType* si) { return si + 1; }
inline const LongType* strideOf(const LongType* si) { return si + 1 + rank(si); }
inline int extraIndex(const LongType* si) { return rank(si) == 0 ? 3 : 2 * rank(si) + 1; }
inline LongType extra(const LongType* si) { return si[extraIndex(si)]; }
inline LongType ews(const LongType* si) { return si[shapeInfoLength(rank(si)) - 2]; }
inline char order(const LongType* si) { return (char)si[shapeInfoLength(rank(si)) - 1]; }
inline bool isEmpty(const LongType* si) { return (extra(si) & ARRAY_EMPTY) != 0; }
inline LongType length(const LongType* si) {
  if (isEmpty(si)) return 0;
  LongType n = 1;
  for (int i = 0; i < rank(si); i++) n *= shapeOf(si)[i];
  return n;
}
LongType flagForDataType(DataType t);
DataType dataType(const LongType* si);  // ArrayOptions::dataTypeValue, libnd4j/include/array/ArrayOptions.hXX:247-271
}  // namespace shape

// Fixed-size shape record handed to kernels by value.
struct DevShape {
  int rank;
  LongType shape[MAX_DEV_RANK];
  LongType stride[MAX_DEV_RANK];
};

}  // namespace nd4jhip
