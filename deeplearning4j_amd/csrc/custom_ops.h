// Registry of declarable ("custom") ops reached through execCustomOp2 / calculateOutputShapes2.
#pragma once
#include <functional>
#include <string>
#include <vector>

#include "kernels.h"
#include "runtime.h"

namespace nd4jhip {
namespace ops {

struct OpDescriptor {
  std::string name;
  LongType hash;
  int nIn, nOut;      // declared arities as the reference registers them (negative = variable)
  bool inplace;
  int nT, nI;
  std::function<void(Context&)> exec;
  std::function<std::vector<std::vector<LongType>>(Context&)> shapeFn;
};

LongType opHash(const std::string& name);  // helpers/impl/helper_hash.cpp:33-70 of the reference
const OpDescriptor* findOp(LongType hash);
const OpDescriptor* findOpByName(const std::string& name);
const char* allCustomOps();                // "name:hash:nIn:nOut:inplace:nT:nI:;" per op (OpRegistrator.cpp:106-125)
void executeOp(const OpDescriptor& op, Context& ctx);

}  // namespace ops

// shared with the legacy facade
void runIndexReduce(const char* fn, int opNum, NDArray* x, NDArray* z, const std::vector<LongType>& dims);
// value reductions and summary statistics behind both the legacy entry points and the reduce_* custom ops
void runReduce(const char* fn, ReduceKind k, NDArray* x, NDArray* z, const std::vector<LongType>& dims);
void runReduceMisc(const char* fn, MiscReduceKind k, NDArray* x, NDArray* z, std::vector<LongType> dims, bool biasCorrected);

}  // namespace nd4jhip
