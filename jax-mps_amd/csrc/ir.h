// In-memory form of a StableHLO module: SSA values with static shapes, ops with
// normalised attributes, single-block regions.  Replaces the mlir::ModuleOp the
// reference keeps alive inside its executable (reference:
// src/pjrt_plugin/mlx_executable.h:62, stablehlo_parser.h:17-44).
#pragma once

#include <cstdint>
#include <cstring>
#include <map>
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

namespace mi355 {

enum class DType : uint8_t { Invalid, Pred, S8, S16, S32, S64, U8, U16, U32, U64, F16, F32, F64, BF16, Token };

inline size_t dtypeSize(DType d) {
  switch (d) {
    case DType::Pred: case DType::S8: case DType::U8: return 1;
    case DType::S16: case DType::U16: case DType::F16: case DType::BF16: return 2;
    case DType::S32: case DType::U32: case DType::F32: return 4;
    case DType::S64: case DType::U64: case DType::F64: return 8;
    default: return 0;
  }
}
inline bool isFloat(DType d) { return d == DType::F16 || d == DType::F32 || d == DType::F64 || d == DType::BF16; }
inline bool isUnsigned(DType d) { return d == DType::U8 || d == DType::U16 || d == DType::U32 || d == DType::U64 || d == DType::Pred; }
inline bool isSignedInt(DType d) { return d == DType::S8 || d == DType::S16 || d == DType::S32 || d == DType::S64; }
inline bool isInt(DType d) { return isSignedInt(d) || (isUnsigned(d) && d != DType::Pred); }
const char* dtypeName(DType d);           // "f32", "bf16", "i32", "ui8", "i1"
DType dtypeFromName(const std::string&);  // inverse; Invalid if unknown

struct TensorType {
  DType dt = DType::Invalid;
  std::vector<int64_t> dims;
  int64_t numel() const { int64_t n = 1; for (auto d : dims) n *= d; return n; }
  size_t bytes() const { return (size_t)numel() * dtypeSize(dt); }
  int rank() const { return (int)dims.size(); }
  bool operator==(const TensorType& o) const { return dt == o.dt && dims == o.dims; }
  std::string str() const;
};

struct DenseData {
  TensorType type;
  bool splat = false;
  std::vector<uint8_t> bytes;  // numel*size bytes, or one element if splat
};

struct Attr {
  enum Kind { None, Int, Float, Bool, Str, Ints, Dense, Dict, List, Type } kind = None;
  int64_t i = 0;
  double f = 0;
  bool b = false;
  std::string s;
  std::vector<int64_t> ints;
  std::shared_ptr<DenseData> dense;
  std::map<std::string, Attr> dict;
  std::vector<Attr> list;
  TensorType type;
};

struct Op;
struct Region;

struct Value {
  int id = -1;
  TensorType type;
  Op* def = nullptr;       // null for region arguments
  int defIndex = 0;        // result index in def, or argument index
  Region* argOf = nullptr; // region whose argument this is
  std::string name;        // textual name, for diagnostics
  std::vector<Op*> users;  // filled by Module::rebuildUses
};

struct ConvDims {
  int lhsBatch = 0, lhsFeature = 0; std::vector<int> lhsSpatial;
  int rhsIn = 0, rhsOut = 0; std::vector<int> rhsSpatial;
  int outBatch = 0, outFeature = 0; std::vector<int> outSpatial;
};

struct Region {
  std::vector<std::unique_ptr<Value>> args;
  std::vector<std::unique_ptr<Op>> ops;  // last op is the terminator ("return")
  Op* parent = nullptr;
  Op* terminator() const { return ops.empty() ? nullptr : ops.back().get(); }
};

struct Op {
  std::string name;  // without the "stablehlo." prefix: "add", "dot_general", "return", "call", ...
  std::vector<Value*> operands;
  std::vector<std::unique_ptr<Value>> results;
  std::map<std::string, Attr> attrs;
  std::vector<std::unique_ptr<Region>> regions;
  Region* parent = nullptr;
  int line = 0;
  bool dead = false;

  bool has(const std::string& k) const { return attrs.count(k) != 0; }
  const std::vector<int64_t>& ints(const std::string& k) const {
    static const std::vector<int64_t> empty;
    auto it = attrs.find(k);
    return it == attrs.end() ? empty : it->second.ints;
  }
  int64_t integer(const std::string& k, int64_t dflt = 0) const {
    auto it = attrs.find(k);
    return it == attrs.end() ? dflt : it->second.i;
  }
  const std::string& str(const std::string& k) const {
    static const std::string empty;
    auto it = attrs.find(k);
    return it == attrs.end() ? empty : it->second.s;
  }
  Value* result(int i = 0) const { return results[i].get(); }
  ConvDims convDims;  // for "convolution"
};

struct Func {
  std::string name;
  bool isPublic = false;
  Region body;
  std::vector<TensorType> resultTypes;
  // per argument: >= 0 the result the argument's buffer may be reused for (`tf.aliasing_output = k`), -2 a donor
  // without a fixed result (`jax.buffer_donor = true`), -1 neither
  std::vector<int> argDonation;
};

struct Module {
  std::vector<std::unique_ptr<Func>> funcs;
  int64_t numPartitions = 1, numReplicas = 1;   // mhlo.num_partitions / mhlo.num_replicas of the module (1 when absent)
  Func* find(const std::string& name) const {
    for (auto& f : funcs) if (f->name == name) return f.get();
    return nullptr;
  }
  Func* main() const { return find("main"); }
};

struct CompileError : std::runtime_error {
  using std::runtime_error::runtime_error;
};

// Front end: program bytes -> Module.  The bytes are StableHLO text or an MLIR bytecode file holding a VHLO portable
// artifact (rewritten to text first, bytecode.cc).  Throws CompileError with a line number.
std::unique_ptr<Module> parseStableHLOText(const char* data, size_t size);
bool isMlirBytecode(const char* data, size_t size);
std::string vhloBytecodeToStableHLOText(const char* data, size_t size);

// Passes (passes.cc, fused_calls.cc)
void lowerFusedOpCalls(Module& m);   // custom_call @mps.sdpa / rms_norm / layer_norm / rope / gelu and their backward forms -> calls of StableHLO functions
void inlineCalls(Module& m);          // replaces every "call" by the callee body
void lowerIntegerDots(Module& m);    // integer / boolean dot_general -> broadcast, multiply, reduce
void lowerSingleDeviceOps(Module& m);  // one-device all_reduce -> operands, partition_id / replica_id -> 0, tokens -> f32 scalar placeholders
void reluMasksFromActivations(Module& m);  // compare(v, 0, GT) beside maximum(v, 0) reads the maximum instead
void lowerTopK(Module& m);           // chlo.top_k -> stable descending sort of (value, position) + slice
void lowerBitcastWidths(Module& m);      // bitcast_convert between types of different width -> shifts and same-width bitcasts
void widenScatterTypes(Module& m);       // scatter on bool / 8- and 16-bit integers / f16 -> on the 32-bit type that holds them
void widenHalfProducts(Module& m);       // f16 dot_general / convolution -> f32 product between converts
void canonicalizeDotLayouts(Module& m);  // dot_general whose operand dims do not collapse to strided matrices: transposes in front
void lowerEmptyReductions(Module& m);   // reduce over zero elements -> broadcast of the init values
void lowerRng(Module& m);            // rng_bit_generator -> counter update + threefry2x32 as plain ui32 ops
void lowerWindowOps(Module& m);      // reduce_window / select_and_scatter with small windows -> pad, strided slices, elementwise ops
void lowerGeneralScatters(Module& m); // scatter forms other than whole rows along dim 0 -> element scatter with computed keys
void eliminateDeadCode(Region& r);    // removes ops whose results are unused (recursively)
void rebuildUses(Region& r);          // recompute Value::users for a region tree
void checkSupported(const Module& m); // throws CompileError naming unsupported ops
int countOps(const Region& r);

// Loop analysis shared by the passes and the planner (hoist.cc)
bool constantInt(Value* v, int64_t& out);   // the value of a compile-time constant integer scalar
struct LoopCounter { int carry = -1; int64_t init = 0, step = 0; };
// iterations of a `while` whose condition compares one carry with a constant and whose body steps that carry by a
// constant from a constant start; -1 when the count is not static.  `counter` (optional) receives the carry.
int64_t staticTripCount(Op* whileOp, LoopCounter* counter = nullptr);
// inside counted loops, a product of a loop-invariant operand with the counter-selected slice of a loop-invariant tensor
// becomes one product over the whole tensor ahead of the loop, and the body slices its result
void hoistLoopProducts(Module& m);
// updates = select(index in range, u, 0) ahead of a whole-row scatter with that index: the scatter reads u (rows out of
// range are dropped by the scatter itself)
void dropScatterIndexMasks(Module& m);

}  // namespace mi355
