// Execution plan: what PJRT_Client_Compile produces from a StableHLO module and
// what PJRT_LoadedExecutable_Execute replays.  A plan is a list of steps over
// statically assigned buffers; there is no per-call graph walk (the reference
// re-dispatches ops through a string-keyed handler table on the first call and
// replays an MLX-compiled graph afterwards, src/pjrt_plugin/mlx_executable.cc:799-1008).
#pragma once

#include <cstdint>
#include <memory>
#include <string>
#include <unordered_map>
#include <vector>

#include "hip_abi.h"
#include "ir.h"

namespace mi355 {

// Where a materialised value lives during one execution.
struct BufRef {
  enum Kind : uint8_t { None, Param, Output, Temp, Const } kind = None;
  int index = 0;       // parameter / output number
  int64_t offset = 0;  // byte offset inside the arena (Temp) or the constant pool (Const)
  // Inside a counted loop whose counter the host follows (Step::hostCounter): the address moves with the iteration,
  // by CompiledProgram::ivTables[ivTable][k] bytes at iteration k of the loop at nesting depth ivDepth.  That is how a
  // kernel reads the counter (a table of its values in the constant pool) and how a product reads xs[i] in place.
  int ivTable = -1;
  int ivDepth = 0;
  bool operator==(const BufRef& o) const { return kind == o.kind && index == o.index && offset == o.offset && ivTable == o.ivTable; }
  bool operator!=(const BufRef& o) const { return !(*this == o); }
};

// One generated (runtime-compiled) kernel; identical sources are shared.
struct GenKernel {
  std::string name;
  std::string source;
  void* function = nullptr;  // hipFunction_t once loaded
};

struct GemmDesc {   // C[b0,b1] = A[b0,b1] x B[b0,b1]; operands addressed through element strides, C dense row-major
  int64_t batch0 = 1, batch1 = 1, M = 0, N = 0, K = 0;
  int64_t aB0 = 0, aB1 = 0, aRow = 0, aCol = 0;   // A(m,k) = a[b0*aB0 + b1*aB1 + m*aRow + k*aCol]
  int64_t bB0 = 0, bB1 = 0, bRow = 0, bCol = 0;   // B(k,n) = b[b0*bB0 + b1*bB1 + k*bRow + n*bCol]
  DType inType = DType::F32, outType = DType::F32;
  int act = 0;                                     // 1: tanh-form GELU epilogue with the constants below; 2: maximum(x, 0)
  float actA = 0.f, actB = 0.f, actC = 0.f;
};

struct ConvDesc {   // StableHLO convolution with arbitrary dimension numbers (<= 3 spatial dims, kernels specialise 2)
  int nsp = 2;
  int64_t N = 0, C = 0, O = 0;             // batch (per batch group), input features (total), output features
  int64_t in[3] = {1, 1, 1}, k[3] = {1, 1, 1}, out[3] = {1, 1, 1};
  int64_t stride[3] = {1, 1, 1}, padLo[3] = {0, 0, 0}, ldil[3] = {1, 1, 1}, rdil[3] = {1, 1, 1};
  int64_t rev[3] = {0, 0, 0};
  int64_t featureGroups = 1, batchGroups = 1;
  // element strides of each logical dim in the three tensors
  int64_t lhsB = 0, lhsF = 0, lhsS[3] = {0, 0, 0};
  int64_t rhsI = 0, rhsO = 0, rhsS[3] = {0, 0, 0};
  int64_t outB = 0, outF = 0, outS[3] = {0, 0, 0};
  DType type = DType::F32;
};

struct ScatterDesc {   // row scatter: operand [rows, rowSize...], one index per update row
  int64_t numUpdates = 0, rowElems = 0, operandRows = 0;
  int kind = 0;        // 0 add, 1 set, 2 mul, 3 min, 4 max
  DType type = DType::F32, indexType = DType::S32;
  bool fill = false;   // the operand is a splat that the scatter writes itself (no buffer holds it beforehand)
  uint32_t fillBits = 0;
};

struct AttentionDesc {   // softmax(scale * Q K^T, masked -> `masked`) V, tensors addressed as [b, n, t|s, h] through element strides
  int64_t B = 0, N = 0, T = 0, S = 0, H = 0;
  int64_t qB = 0, qN = 0, qT = 0, kB = 0, kN = 0, kS = 0, vB = 0, vN = 0, vS = 0, oB = 0, oN = 0, oT = 0, mB = 0, mN = 0, mT = 0, mS = 0;
  float scale = 1.f, masked = 0.f;
  bool hasMask = false;
};

struct Plan;

struct Step {
  enum Kind { Kernel, Gemm, Conv, ScatterRows, Copy, Fill, While, Case, GemmGroup, Attention, FlagInit, FlagAnd } kind = Kernel;
  std::string label;  // op name(s) for profiling ranges and error messages

  // Kernel
  int kernel = -1;
  unsigned grid[3] = {1, 1, 1}, block[3] = {1, 1, 1};
  std::vector<BufRef> args;        // pointer arguments, in kernel order
  int64_t algoBytes = 0;           // distinct input bytes + output bytes (for bandwidth reports)
  std::vector<uint8_t> argWrites;  // planning only: 1 where the kernel writes the argument's buffer
  int time = 0;                    // planning only: position in the buffer-lifetime clock

  // Gemm / Conv / ScatterRows
  GemmDesc gemm;
  AttentionDesc attn;              // Attention: args = [q, k, v, out, (mask)]
  GemmDesc gemm2;                  // dual: second product summed into the same result; args = [a, b, c, a2, b2]
  bool dual = false;
  std::vector<Step> parts;         // GemmGroup: independent small products launched together (each a Gemm step)
  ConvDesc conv;
  ScatterDesc scatter;
  BufRef bias;                     // Gemm: per-column values added to the product (kind None: no bias)
  BufRef addend;                   // Gemm (small fp32 products): a tensor of the result's shape added to the product (kind None: none)
  int statsArg = -1;               // Conv: index in args of the column-sum buffer (the sum-of-squares buffer follows), or -1
  // A step whose results nothing needs for a while (a filter gradient, read only by the optimizer update at the end of
  // the step) may run on a second stream next to the steps that follow it: forkId >= 0 marks it, and the first later
  // step that touches what it wrote, or writes what it read, lists the id in `joins` and waits for it.
  int forkId = -1;
  std::vector<int> joins;
  int64_t workspaceOffset = -1;    // arena offset of split-K / sort scratch
  int64_t workspaceBytes = 0;
  int splitK = 1;

  // Copy / Fill.  A Copy with `copyBytes` set moves several disjoint buffers in one launch:
  // args = [src0, dst0, src1, dst1, ...], copyBytes[i] = size of pair i.
  BufRef src, dst;
  int64_t bytes = 0;
  std::vector<int64_t> copyBytes;
  // Conditional copy, decided on the device (no host read-back): condMode 1 copies while the loop flag at condBuf is
  // set; condMode 2 copies when the branch index at condBuf (type condType) selects branch condWant of condCount.
  BufRef condBuf;
  int condMode = 0;
  DType condType = DType::S32;
  int64_t condWant = 0, condCount = 0;

  // While / Case
  std::unique_ptr<Plan> cond;                 // While: evaluates the predicate into predBuf
  std::vector<std::unique_ptr<Plan>> bodies;  // While: [body]; Case: branches
  BufRef predBuf;                             // i1 (While) or i32 index (Case)
  int64_t tripCount = -1;                     // >= 0 when the loop is counted and the count is static
  // Counted loop whose counter carry is never computed on the device: iteration k reads entry k of a table of the
  // counter's values, and operands sliced at the counter are addressed by the host (BufRef::ivTable).
  bool hostCounter = false;
  int ivDepth = 0;
  DType predType = DType::Pred;
  // Dynamic While: the loop's alive flag (one int on the device).  Iterations run in chunks without host
  // round trips: each evaluates the condition, folds it into the flag (FlagAnd), runs the body into temporaries and
  // commits the carries with copies conditional on the flag; the host reads the flag once per chunk.
  // FlagInit: flagBuf = parentFlag (kind None: 1).  FlagAnd: flagBuf &= predBuf.
  // Case with `predicated`: every branch runs and the result copies are conditional on the index (no host read).
  BufRef flagBuf, parentFlag;
  bool predicated = false;
};

struct Plan {
  int numForks = 0;                 // forked steps of this (top-level) plan; those nobody joined are joined at its end
  std::vector<Step> steps;
};

struct OutputInfo {
  TensorType type;
};

struct CompiledProgram {
  std::unique_ptr<Module> module;
  Plan plan;
  std::vector<GenKernel> kernels;
  std::vector<TensorType> paramTypes;
  std::vector<int> paramDonation;   // per parameter: -1 not donated by the program, otherwise donated (>= 0: to that result)
  std::vector<OutputInfo> outputs;
  std::vector<uint8_t> constPool;   // host image of the constant pool
  std::vector<std::vector<int64_t>> ivTables;   // per-iteration byte offsets of references that follow a host-side loop counter
  int64_t arenaBytes = 0;
  int numOps = 0, numSteps = 0;
  std::string dump;                 // human-readable plan (MI355X_DUMP_PLAN)
};

// planner.cc
std::unique_ptr<CompiledProgram> compileProgram(std::unique_ptr<Module> module);
int abiDtypeCode(DType d);   // element type code of the C-ABI kernel entry points (-1: not supported there)
mi355_conv_desc toAbi(const ConvDesc& c);
mi355_gemm_desc toAbi(const GemmDesc& g);
mi355_attention_desc toAbi(const AttentionDesc& a);

}  // namespace mi355
