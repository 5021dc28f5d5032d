// HIP source generation for fused kernels.
//
// A fusion group is a root (an elementwise/indexing value that has to be written
// to memory, a dynamic_update_slice window, or one or more sibling reductions)
// plus every producer that is cheap enough to recompute per element.  The
// generator walks the group once per output element *symbolically* and prints a
// kernel in which broadcasts, transposes, slices, pads, concatenations, iota,
// gather and dynamic_slice are index arithmetic, never copies.
#pragma once

#include <functional>
#include <string>
#include <vector>

#include <cstdlib>

#include "ir.h"

namespace mi355 {

// MI355X_STRICT_BF16=1: every 16-bit float op rounds its result as the program's types say, and the fusions that move
// a rounding point (activation in the GEMM epilogue, the one-launch attention kernel) are off.  Read at every compile.
inline bool strictBf16() {
  const char* e = getenv("MI355X_STRICT_BF16");
  return e && e[0] == '1';
}


struct KArg {
  enum Kind { In, Out, Work } kind = In;
  Value* value = nullptr;   // In: materialised leaf; Out: root value
  int64_t workOffset = 0;   // Work: byte offset inside the step's workspace
};

struct Launch {
  std::string source;       // complete translation unit; entry point is always `k`
  unsigned grid[3] = {1, 1, 1};
  unsigned block[3] = {1, 1, 1};
  std::vector<KArg> args;
};

struct FusedCode {
  std::vector<Launch> launches;
  int64_t workspaceBytes = 0;
  bool epilogueFused = false;
  std::vector<Value*> leaves;   // distinct materialised inputs
  std::vector<int64_t> partialOffsets;
  bool sideStored = false;          // the side stores asked for are written by the first launch (extra Out arguments)   // generateReduceKernel with external partials: where each reduction's partial sums sit in the workspace
};

using LeafPredicate = std::function<bool(Value*)>;

// out[i] = f(leaves...) for every element of `root`.
FusedCode generateLoopKernel(Value* root, const LeafPredicate& isLeaf);
FusedCode generateLoopKernel(const std::vector<Value*>& roots, const LeafPredicate& isLeaf);

// stablehlo.reduce with several inputs and/or an arbitrary reducer region (argmax, argmin, ...).
FusedCode generateRegionReduce(Op* reduce, const LeafPredicate& isLeaf);

// Reductions over the trailing dims in dependency phases plus the elementwise values that
// consume them, computed row by row in one kernel.
struct RowProgram {
  std::vector<std::vector<Op*>> phases;   // phase p may read the results of phases < p
  std::vector<Value*> fullRoots;          // stored values of the unreduced shape
  std::vector<Value*> keptRoots;          // stored values of the reduced (per-row) shape
};
FusedCode generateRowProgram(const RowProgram& rp, const LeafPredicate& isLeaf);

// In-place window write of a dynamic_update_slice: iterates over the update
// tensor and stores into `dus` result storage (which already holds the operand).
FusedCode generateDusKernel(Op* dus, const LeafPredicate& isLeaf);

// stablehlo.sort of a dim that fits LDS (sortLdsBytes <= 60 KiB): one workgroup per slice, comparator region compiled.
// All operands must be in memory.
int64_t sortLdsBytes(Op* sort);
FusedCode generateSortKernel(Op* sort, const LeafPredicate& isLeaf);

// Several independent kernels with one-dimensional grids as the segments of one launch: block b
// runs the kernel whose block range holds b.  Arguments are the kernels' arguments, concatenated.
// Returns "" when one of the sources cannot take part (batchableKernel is the cheap test).
bool batchableKernel(const std::string& source);
std::string combineKernels(const std::vector<const std::string*>& sources, const std::vector<unsigned>& gridX);

// One or more stablehlo.reduce ops with identical input shape and dimensions.
// Returns false in `ok` when a reducer body is not a single add/mul/max/min/and/or.
// `epilogue`: values of the result shape computed from the results (and other inputs of that shape); they are
// produced by the pass that folds partial sums when there is one (FusedCode::epilogueFused), otherwise ignored.
// `externalPartials` > 0: the partial results (that many per output, float accumulators, partial p of output k at
// [k * externalPartials + p] from partialOffsets[j] of the workspace) are written by an earlier step; only the folding pass is generated.
// `sideStores`: values of the input's shape that the reductions' inputs are computed from and that are needed in memory too:
// the pass over the data writes them while it reduces (each element is visited exactly once), so no kernel of their own
// stores them and the reduction does not read them back.  Only honoured by the column-style kernel (FusedCode::sideStored).
FusedCode generateReduceKernel(const std::vector<Op*>& reduces, const LeafPredicate& isLeaf, const std::vector<Value*>& epilogue = {}, int64_t externalPartials = 0,
                               const std::vector<Value*>& sideStores = {});
// the kernel generateReduceKernel would choose walks the reduced dims with the kept ones across the lanes (column style)
bool reduceIsColumnStyle(const Op* reduce);
// column reductions over at most this many input elements run as one launch of a few workgroups
int64_t reduceOnePassLimit();

// True if codegen can inline `op` into a consumer (elementwise / indexing ops).
bool isFusibleOp(const Op& op);
// True if the reducer body of `reduce` is one supported binary op.
bool isSimpleReduce(const Op& reduce);
const char* simpleReduceKind(const Op& reduce);   // "add", "maximum", ... for a one-input reduce with a single-op reducer, else null

}  // namespace mi355
