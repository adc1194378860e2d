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

// ---- recorded op sequences --------------------------------------------------------------------------------------------
// While a stream capture is open the facade also notes every op call it recognises (what was called, on which arrays, with
// which arguments, and a closure that runs it as the eager call does).  When every call of the capture was recognised,
// the sequence is replayed through fuseRecordedOps before the graph is instantiated: neighbouring ops that one kernel can
// serve are merged (a pairwise Add and the layer_norm of its result; xw_plus_b and the GELU transform / the column-slice
// assigns that follow it), every merged kernel writing exactly what the separate ops would have written, bit for bit.
struct RecordedOp {
  enum Kind { CUSTOM, PAIRWISE, TRANSFORM_STRICT, TRANSFORM_ANY, RAW } kind = CUSTOM;   // RAW: a copy or fill on plain device pointers (memcpyAsync / memsetAsync), never merged
  const ops::OpDescriptor* op = nullptr;   // CUSTOM
  Context ctx;                             // CUSTOM: copy of the caller's argument bag (arrays borrowed)
  int opNum = 0;                           // legacy loops
  NDArray *x = nullptr, *y = nullptr, *z = nullptr;
  std::function<void(const RecordedOp&)> run;   // legacy loops: executes the op on this record's arrays exactly as the eager call does
  // adopt() replaces every array above by a copy of the view held here (same buffer, offset, shape and strides; the
  // buffer is shared).  The facade calls it the moment the op is recorded, so neither the merging pass nor a replay
  // depends on how long the caller keeps its array handles.
  std::vector<std::shared_ptr<NDArray>> owned;
  void adopt();
};
// The launch plan of the sequence; nFused counts the ops that the plan gives to a neighbour's kernel.  A step may still
// run its ops separately when the kernel declines the operands it meets at run time: fusedAppliedCounter() is raised by
// every op whose work did run inside a neighbour's kernel (the caller zeroes it before running a plan).
std::vector<std::function<void()>> fuseRecordedOps(std::vector<RecordedOp>& ops, int& nFused);
int& fusedAppliedCounter();

// shared with the legacy facade
void runIndexReduce(const char* fn, int opNum, NDArray* x, NDArray* z, const std::vector<LongType>& dims);
// value reductions and summary statistics behind both the legacy entry points and the reduce_* custom ops
void runReduce(const char* fn, ReduceKind k, NDArray* x, NDArray* z, const std::vector<LongType>& dims);
void runReduceMisc(const char* fn, MiscReduceKind k, NDArray* x, NDArray* z, std::vector<LongType> dims, bool biasCorrected, double param = 0.0);

}  // namespace nd4jhip
