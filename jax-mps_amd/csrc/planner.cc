// StableHLO module -> execution plan.
//
//  1. decide which values are written to memory (everything else is recomputed
//     inside the kernel that needs it),
//  2. emit one step per materialised root in program order (generated fused
//     kernels, GEMM / convolution / row-scatter library steps, loops, branches),
//  3. assign every temporary a fixed offset in one arena by liveness.
//
// The chains that end up fused are the ones the reference's pattern pass names
// (bias-add, softmax, LayerNorm, RMSNorm: src/pjrt_plugin/passes/*.cc) plus
// whatever else is elementwise; nothing here is pattern-matched by name.
#include <algorithm>
#include <array>
#include <cstring>
#include <functional>
#include <cmath>
#include <set>
#include <sstream>
#include <unordered_map>
#include <unordered_set>

#include "codegen.h"
#include "hip_abi.h"
#include "plan.h"

namespace mi355 {

namespace {

constexpr int64_t kSmallNumel = 8192;   // values at most this big are never materialised just to avoid recomputation
// Inside a loop body a launch costs more than any amount of arithmetic on a tensor this small, and a kernel that
// recomputes what a neighbour also computes does not have to wait for it: the two can share a launch.
constexpr int64_t kLoopSmallNumel = 131072;
constexpr int64_t kAlign = 256;

struct Storage {
  BufRef::Kind kind = BufRef::Temp;
  int index = 0;          // param / output number
  int64_t bytes = 0;
  int64_t offset = -1;    // arena or const-pool offset
  int first = -1, last = -1;
  std::vector<int> uses;
  int values = 0;         // SSA values bound to this storage
  int ivTable = -1;       // references move with the iteration of a host-counted loop (BufRef::ivTable)
  int ivDepth = 0;
  int aliasOf = -1;       // a window of another storage (the halves of a double-buffered loop carry): no memory of its own
  int64_t aliasOffset = 0;
};

bool isExpensive(const std::string& n) {
  static const std::set<std::string> s = {"exponential", "exponential_minus_one", "log", "log_plus_one", "tanh", "tan",
                                          "sine", "cosine", "logistic", "power", "atan2", "cbrt", "remainder", "gather"};
  return s.count(n) != 0;
}

bool isPassThrough(const Op& op) {
  return op.name == "optimization_barrier" || op.name == "custom_call";
}

class Planner {
 public:
  explicit Planner(CompiledProgram& p) : P(p) {}

  void run() {
    Func* main = P.module->main();
    Region& body = main->body;
    ivArgs().clear();
    rebuildUses(body);
    for (auto& a : body.args) {
      P.paramTypes.push_back(a->type);
      int sid = newStorage(a->type.bytes(), BufRef::Param, (int)P.paramTypes.size() - 1);
      bind(a.get(), sid);
    }
    analyze(body);
    emitRegion(body, P.plan);
    // program outputs
    Op* ret = body.terminator();
    int t = ++time_;
    for (size_t k = 0; k < ret->operands.size(); ++k) {
      Value* v = ret->operands[k];
      OutputInfo oi;
      oi.type = v->type;
      P.outputs.push_back(oi);
      int sid = storageOf(v);
      Storage& s = st_[sid];
      if (s.kind == BufRef::Temp && !boundToOutput_.count(sid)) {
        s.kind = BufRef::Output;
        s.index = (int)k;
        boundToOutput_.insert(sid);
      } else {
        int out = newStorage(v->type.bytes(), BufRef::Output, (int)k);
        Step c;
        c.kind = Step::Copy;
        c.label = "copy-to-output";
        c.src = ref(sid, t);
        c.dst = ref(out, t);
        c.bytes = (int64_t)v->type.bytes();
        P.plan.steps.push_back(std::move(c));
      }
    }
    static const bool batching = !getenv("MI355X_BATCH_KERNELS") || atoi(getenv("MI355X_BATCH_KERNELS")) != 0;
    groupSmallGemms(P.plan);
    if (batching) sinkKernelsInLoops(P.plan, false);
    if (batching) batchKernels(P.plan);
    forkDistantConvolutions(P.plan);
    assignArena();
    patch(P.plan);
    P.numSteps = countSteps(P.plan);
    P.numOps = countOps(body);
    if (getenv("MI355X_DUMP_PLAN")) dumpPlan(P.plan, 0);
  }

 private:
  CompiledProgram& P;
  std::vector<Storage> st_;
  std::unordered_map<Value*, int> storage_;
  std::unordered_map<Value*, bool> needMat_;
  std::unordered_set<Value*> inlineAnyway_;   // stored for a consumer that needs memory, yet cheap enough that kernels recompute it
  std::unordered_map<std::string, int> kernelIds_;
  std::unordered_set<int> boundToOutput_;
  std::vector<std::pair<int, int>> loops_;
  std::unordered_set<Op*> emitted_;
  std::unordered_set<Value*> deferred_;   // values whose own kernel is held back: the reduction that reads them first stores them on the way
  std::unordered_map<Op*, Op*> heldDots_;   // later product of add(dot, dot) -> the earlier one waiting for it
  int time_ = 0;
  // Regions that may execute speculatively (the body of a dynamic loop past its last iteration, the branches of a
  // case that runs all of them and keeps one result) must leave every buffer defined outside them untouched: inside,
  // no value is updated in place in a storage older than the region (ids below the floor).
  std::vector<int> specFloors_;
  std::vector<int> aliveFlags_;   // flag storages of the enclosing dynamic loops
  int loopDepth_ = 0;
  bool outerStorage(int sid) const { return !specFloors_.empty() && sid < specFloors_.back(); }

  // ---------------------------------------------------------------- storages
  int newStorage(size_t bytes, BufRef::Kind kind = BufRef::Temp, int index = 0) {
    Storage s;
    s.kind = kind;
    s.index = index;
    s.bytes = (int64_t)std::max<size_t>(bytes, 4);
    st_.push_back(s);
    return (int)st_.size() - 1;
  }
  void bind(Value* v, int sid) {
    storage_[v] = sid;
    st_[sid].values++;
  }
  bool hasStorage(Value* v) const { return storage_.count(v) != 0; }
  int storageOf(Value* v) {
    auto it = storage_.find(v);
    if (it == storage_.end()) throw CompileError("internal: value " + v->name + " has no storage");
    return it->second;
  }
  // a storage that names `bytes` of `parent` from `offset` on, optionally moving with a host-counted loop's iteration
  int newAlias(int parent, int64_t offset, int64_t bytes, int ivTable) {
    int sid = newStorage((size_t)bytes);
    st_[sid].aliasOf = parent;
    st_[sid].aliasOffset = offset;
    st_[sid].ivTable = ivTable;
    boundToOutput_.insert(sid);     // never turned into an output buffer or taken over as another loop's slot
    return sid;
  }
  BufRef ref(int sid, int t) {
    if (st_[sid].aliasOf >= 0) {    // the memory is the parent's: its lifetime is what the use extends
      BufRef p = ref(st_[sid].aliasOf, t);
      (void)p;
      BufRef r;
      r.kind = BufRef::Temp;
      r.index = sid;
      r.ivTable = st_[sid].ivTable;
      r.ivDepth = st_[sid].ivDepth;
      return r;
    }
    Storage& s = st_[sid];
    s.uses.push_back(t);
    if (s.first < 0 || t < s.first) s.first = t;
    if (t > s.last) s.last = t;
    BufRef r;
    r.kind = BufRef::Temp;   // patched after arena assignment
    r.index = sid;
    r.ivTable = s.ivTable;
    r.ivDepth = s.ivDepth;
    return r;
  }

  // a reference that follows a view taken at a host-counted loop's counter: byte offsets per iteration
  void followCounter(BufRef& r, const std::vector<int64_t>& iterElems, int64_t elemBytes) {
    if (iterElems.empty()) return;
    std::vector<int64_t> bytes;
    for (auto e : iterElems) bytes.push_back(e * elemBytes);
    P.ivTables.push_back(std::move(bytes));
    r.ivTable = (int)P.ivTables.size() - 1;
    r.ivDepth = 0;
  }

  // ---------------------------------------------------------------- analysis
  static Region* regionOf(Value* v) { return v->def ? v->def->parent : v->argOf; }

  // stablehlo.reverse of a filter over its window dims only: the convolution kernels take a
  // per-dim "window reversal" flag, so the flipped copy is never made
  static bool isWindowReverse(Value* v, Op* conv) {
    if (!v->def || v->def->name != "reverse" || conv->name != "convolution" || conv->operands.size() < 2 || conv->operands[1] != v) return false;
    if (v->users.size() != 1) return false;
    for (auto d : v->def->ints("dims"))
      if (std::find(conv->convDims.rhsSpatial.begin(), conv->convDims.rhsSpatial.end(), d) == conv->convDims.rhsSpatial.end()) return false;
    return true;
  }

  // bit pattern of the element every position of `v` holds, when `v` is a broadcast of a constant
  static bool splatBits(Value* v, uint32_t& bits) {
    Op* d = v->def;
    while (d && (d->name == "broadcast_in_dim" || d->name == "reshape") && d->operands[0]->type.dt == v->type.dt) d = d->operands[0]->def;
    if (!d || d->name != "constant") return false;
    auto& dd = *d->attrs.at("value").dense;
    if ((!dd.splat && dd.type.numel() != 1) || dd.type.dt != v->type.dt) return false;
    const size_t size = dtypeSize(dd.type.dt);
    if ((size != 2 && size != 4) || dd.bytes.size() < size) return false;
    bits = 0;
    memcpy(&bits, dd.bytes.data(), size);
    return true;
  }

  // A splat operand of a scatter that nothing else reads (the zeros a gradient is scattered into) is written by
  // the scatter itself: its fill shares a launch with the sort of the indices.
  static bool scatterWritesSplat(Value* v, Op* user) {
    static const bool on = !getenv("MI355X_SCATTER_FILL") || atoi(getenv("MI355X_SCATTER_FILL")) != 0;
    uint32_t bits;
    return on && user->name == "scatter" && user->operands.size() == 3 && user->operands[0] == v && user->operands[1] != v && user->operands[2] != v &&
           v->users.size() == 1 && user->operands[2]->type.numel() > 0 && splatBits(v, bits);
  }

  static bool forcedBy(Value* v, Op* user) {
    if (isWindowReverse(v, user)) return false;
    if (scatterWritesSplat(v, user)) return false;
    if (dotTakesView(v, user)) return false;
    if (user->name == "gather") return user->operands[0] == v;       // random access needs memory
    if (isFusibleOp(*user)) return false;
    if (user->name == "reduce") return false;   // every reduce kernel evaluates its inputs in place
    if (user->name == "dynamic_update_slice") return user->operands[0] == v;
    return true;
  }

  // `v` is at most `budget` cheap elementwise ops away from values that are in memory whatever the analysis decides
  static bool cheapFromMemory(Value* v, int& budget) {
    Op* d = v->def;
    if (!d || !isFusibleOp(*d) || d->results.size() != 1) return alwaysInMemory(v);
    static const std::set<std::string> cheap = {"add", "subtract", "multiply", "negate", "select", "compare", "and", "or", "not", "convert", "reshape",
                                                "broadcast_in_dim", "constant", "minimum", "maximum", "clamp", "iota"};
    if (!cheap.count(d->name)) return false;
    if (d->name == "constant") {
      auto& dd = *d->attrs.at("value").dense;
      return dd.splat || dd.type.numel() == 1;
    }
    if (d->name != "reshape" && d->name != "broadcast_in_dim" && d->name != "convert" && --budget < 0) return false;
    for (auto* o : d->operands) if (!cheapFromMemory(o, budget)) return false;
    return true;
  }

  void analyze(Region& r) {
    // forward: set of leaves every value depends on (capped)
    std::unordered_map<Value*, std::vector<Value*>> leaves;
    auto addLeaf = [](std::vector<Value*>& dst, Value* l) {
      if (dst.size() < 6 && std::find(dst.begin(), dst.end(), l) == dst.end()) dst.push_back(l);
    };
    for (auto& op : r.ops) {
      for (auto& sub : op->regions) analyze(*sub);
      if (!isFusibleOp(*op) || op->results.size() != 1) continue;
      auto& mine = leaves[op->result()];
      for (auto* o : op->operands) {
        auto it = leaves.find(o);
        if (it == leaves.end()) addLeaf(mine, o);
        else for (auto* l : it->second) addLeaf(mine, l);
      }
    }
    // Small values that a much larger kernel reads through a broadcast (per-channel scales, reciprocal standard
    // deviations, gradient coefficients): recomputing their chain for every element of the large tensor makes a
    // memory-bound kernel arithmetic-bound, while storing them costs a few hundred bytes and usually no launch
    // (they ride in the pass that folds the partial sums they are computed from).
    std::unordered_set<Value*> smallStored;
    {
      static const bool off = getenv("MI355X_STORE_SMALL") && atoi(getenv("MI355X_STORE_SMALL")) == 0;
      std::unordered_map<Value*, int> cost;   // arithmetic between a value and the stored values below it
      auto opCost = [](const std::string& n) {
        if (n == "divide" || n == "sqrt" || n == "rsqrt" || isExpensive(n)) return 100;
        if (n == "constant" || n == "reshape" || n == "broadcast_in_dim" || n == "convert" || n == "transpose" || n == "slice") return 0;
        return 1;
      };
      for (auto& op : r.ops) {
        if (!isFusibleOp(*op) || op->results.size() != 1) continue;
        Value* v = op->result();
        int c = opCost(op->name);
        for (auto* o : op->operands) {
          auto it = cost.find(o);
          if (it != cost.end()) c += it->second;
        }
        c = std::min(c, 10000);
        const int64_t n = v->type.numel();
        bool feedsBig = false;
        if (!off && n >= 2 && n <= kSmallNumel)
          for (Op* u : v->users)
            if (u->name == "broadcast_in_dim" && u->parent == &r && u->result()->type.numel() > kSmallNumel && u->result()->type.numel() >= 16 * n) feedsBig = true;
        if (feedsBig && c >= 100) {   // at least one division, square root or transcendental per element saved
          smallStored.insert(v);
          c = 0;
        }
        cost[v] = c;
      }
    }
    // reverse: materialisation decisions
    // contexts[v]: at how many different positions one generated kernel would evaluate v.  An elementwise reader evaluates
    // its operand where it is evaluated itself (and the generator computes a value once per position), a reader that moves
    // data (reverse, slice, pad, gather ...) at a position of its own.  A chain of such readers doubles the count at
    // every link (v + reverse(v), forty times over, is 2^40 copies of the first value): beyond a few dozen the value
    // is stored instead.
    std::unordered_map<Value*, int64_t> contexts;
    std::unordered_map<Value*, std::vector<Op*>> groups;
    for (int k = (int)r.ops.size() - 1; k >= 0; --k) {
      Op* op = r.ops[k].get();
      if (!isFusibleOp(*op) || op->results.size() != 1) continue;
      Value* v = op->result();
      bool forced = false;
      std::vector<Op*> g;
      auto addGroup = [&](Op* o) { if (g.size() < 4 && std::find(g.begin(), g.end(), o) == g.end()) g.push_back(o); };
      bool nestedUse = false;
      for (Op* u : v->users) {
        if (u->parent != &r) { forced = true; nestedUse = true; continue; }
        if (forcedBy(v, u)) { forced = true; continue; }
        if (u->name == "reduce" || u->name == "dynamic_update_slice") { addGroup(u); continue; }
        Value* ur = u->result();
        if (needMat_[ur]) addGroup(u);
        else for (Op* q : groups[ur]) addGroup(q);
      }
      bool mat = forced || op->has("force_materialize") || smallStored.count(v) != 0;
      if (op->name == "constant") {
        auto& d = *op->attrs.at("value").dense;
        if (!d.splat && d.type.numel() > 1) mat = true;
      }
      int64_t positions = 1;
      {
        int64_t same = 0, moved = 0;
        for (Op* u : v->users) {
          if (u->parent != &r || !isFusibleOp(*u) || u->results.size() != 1) continue;
          auto it = contexts.find(u->result());
          const int64_t cu = it == contexts.end() ? 1 : it->second;
          if (sameShapeElementwise(*u)) same = std::max(same, cu);
          else moved += cu;
        }
        positions = std::max<int64_t>(1, same + moved);
        if (positions > 32 && op->name != "constant" && op->name != "iota" && v->type.numel() > 1) {
          mat = true;
          op->attrs["force_materialize"] = Attr();   // and no kernel that stores it may also compute its readers
        }
      }
      if (!mat && v->type.numel() > (loopDepth_ > 0 ? kLoopSmallNumel : kSmallNumel) && g.size() >= 2) {
        int big = 0;
        for (auto* l : leaves[v]) if (l->type.numel() * 4 >= v->type.numel()) ++big;
        bool expensive = isExpensive(op->name);
        for (auto* o : op->operands) if (o->def && !needMat_[o] && isExpensive(o->def->name) && o->def->parent == &r) expensive = true;
        // g consumers each re-reading `big` leaves move g*big tensors; materialising moves big + 1 + g and costs a launch
        static const int limit = getenv("MI355X_RECOMPUTE_LIMIT") ? atoi(getenv("MI355X_RECOMPUTE_LIMIT")) : 1;
        if ((big >= 2 && ((int)g.size() - 1) * (big - 1) > limit) || expensive) mat = true;
      }
      contexts[v] = mat ? 1 : positions;
      needMat_[v] = mat;
      // A small value that a scatter, gather or the like needs in memory, a few integer or select ops away from
      // buffers that exist anyway (normalised indices, say): the kernels that also read it recompute it, so they do
      // not depend on the kernel that stores it and can share its launch.
      static const bool inlineSmall = !getenv("MI355X_INLINE_SMALL") || atoi(getenv("MI355X_INLINE_SMALL")) != 0;
      // (not the sum a product writes together with its bias: the bare product it would be recomputed from is never stored)
      if (inlineSmall && mat && forced && !nestedUse && loopDepth_ == 0 && !op->has("force_materialize") && v->type.numel() <= kSmallNumel && v->users.size() >= 2 &&
          !alwaysInMemory(v)) {
        int budget = 8;
        if (cheapFromMemory(v, budget)) inlineAnyway_.insert(v);
      }
      // in a loop body the same holds for somewhat larger values (cheap chains only: a column reduction runs few
      // workgroups, and each lane would walk an expensive chain once per row)
      if (inlineSmall && mat && forced && !nestedUse && loopDepth_ > 0 && specFloors_.empty() && !op->has("force_materialize") &&
          v->type.numel() <= kLoopSmallNumel && v->users.size() >= 2 && op->name != "constant" && op->name != "dynamic_update_slice" && !alwaysInMemory(v)) {
        int budget = 16;
        if (cheapFromMemory(v, budget)) inlineAnyway_.insert(v);
      }
      if (mat) { g.clear(); g.push_back(op); }
      groups[v] = g;
    }
  }

  // ---------------------------------------------------------------- emission
  LeafPredicate leafPred() {
    return [this](Value* v) { return storage_.count(v) != 0 && !inlineAnyway_.count(v); };
  }

  int kernelId(const std::string& source) {
    auto it = kernelIds_.find(source);
    if (it != kernelIds_.end()) return it->second;
    GenKernel k;
    k.name = "k";
    k.source = source;
    P.kernels.push_back(std::move(k));
    int id = (int)P.kernels.size() - 1;
    kernelIds_[source] = id;
    return id;
  }

  // a convolution step that writes the partial sums a folding kernel reads: its statistics land in that kernel's workspace
  struct ProducerStats { size_t step = 0; int64_t sumOffset = 0, sqOffset = 0; };

  void addFused(Plan& plan, const FusedCode& fc, const std::string& label, const std::vector<Value*>& outs, const ProducerStats* producer = nullptr) {
    int ws = -1;
    int t0 = time_ + 1;
    int t1 = time_ + (int)fc.launches.size();
    if (fc.workspaceBytes > 0) {
      ws = newStorage((size_t)fc.workspaceBytes);
      ref(ws, t0);
      ref(ws, t1);
      st_[ws].uses.clear();
    }
    if (producer) {
      // (before any step is appended: the reference into plan.steps does not survive a push_back)
      Step& cs = plan.steps[producer->step];
      cs.statsArg = (int)cs.args.size();
      BufRef a = ref(ws, cs.time), b = ref(ws, cs.time);
      a.offset = producer->sumOffset;
      b.offset = producer->sqOffset;
      cs.args.push_back(a);
      cs.args.push_back(b);
      cs.label += " + column statistics";
      st_[ws].uses.clear();
    }
    int64_t bytes = 0;
    for (auto* l : fc.leaves) bytes += (int64_t)l->type.bytes();
    for (auto* o : outs) bytes += (int64_t)o->type.bytes();
    for (auto& l : fc.launches) {
      int t = ++time_;
      Step s;
      s.kind = Step::Kernel;
      s.label = label;
      s.kernel = kernelId(l.source);
      for (int d = 0; d < 3; ++d) { s.grid[d] = l.grid[d]; s.block[d] = l.block[d]; }
      for (auto& a : l.args) {
        if (a.kind == KArg::Work) {
          BufRef r = ref(ws, t);
          r.offset = a.workOffset;   // added to the storage offset when patched
          s.args.push_back(r);
        } else {
          s.args.push_back(ref(storageOf(a.value), t));
        }
        s.argWrites.push_back(a.kind != KArg::In);
      }
      s.time = t;
      s.algoBytes = bytes;
      bytes = 0;   // the traffic of a multi-launch reduction is counted once
      plan.steps.push_back(std::move(s));
    }
  }

  // constant scalar value of an i32/i64/etc. value if it is a compile-time constant
  static bool constInt(Value* v, int64_t& out) { return constantInt(v, out); }

  void emitRegion(Region& r, Plan& plan) {
    // attention chains: everything between the two products is skipped, the second product emits the fused step
    std::unordered_map<Op*, AttnMatch> attention;   // keyed by the second product
    std::unordered_set<Op*> attentionInner;
    for (auto& o : r.ops) {
      AttnMatch m;
      if (o->name == "dot_general" && matchAttention(o.get(), m)) {
        bool fresh = true;
        for (Op* a : m.absorbed) if (attentionInner.count(a)) fresh = false;
        if (!fresh) continue;
        for (Op* a : m.absorbed) if (a != m.pv) attentionInner.insert(a);
        attention[o.get()] = m;
      }
    }
    for (size_t pos = 0; pos < r.ops.size(); ++pos) {
      Op* op = r.ops[pos].get();
      if (emitted_.count(op)) continue;
      if (attentionInner.count(op)) continue;
      {
        auto am = attention.find(op);
        if (am != attention.end()) {
          if (emitAttention(am->second, plan)) continue;
          // not eligible after all: emit the chain the ordinary way, in program order, then this product
          for (size_t q = 0; q < pos; ++q) {
            Op* inner = r.ops[q].get();
            if (std::find(am->second.absorbed.begin(), am->second.absorbed.end(), inner) == am->second.absorbed.end()) continue;
            attentionInner.erase(inner);
            emitOne(inner, r, q, plan);
          }
        }
      }
      emitOne(op, r, pos, plan);
    }
  }

  void emitOne(Op* op, Region& r, size_t pos, Plan& plan) {
    {
      if (emitted_.count(op)) return;
      const std::string& n = op->name;
      if (n == "return") return;
      if (n == "dynamic_slice" && sliceBecomesAlias(op, r)) return;
      if (isFusibleOp(*op) && op->results.size() == 1) {
        Value* v = op->result();
        if (!needMat_[v]) return;
        if (storedByAReduction(op, r, pos)) { deferred_.insert(v); return; }
        emitLoopGroup(op, r, pos, plan);
        return;
      }
      if (isPassThrough(*op)) {   // multi-result barrier: results alias operands
        for (size_t k = 0; k < op->results.size(); ++k) {
          Value* o = op->operands[k];
          if (!hasStorage(o)) materializeNow(o, plan);
          bind(op->results[k].get(), storageOf(o));
        }
        return;
      }
      if (n == "reduce") { if (!tryRowProgram(op, r, pos, plan)) emitReduce(op, r, plan); return; }
      if (n == "dot_general" || n == "dot") {
        // add(dot, dot): the earlier product waits for the later one when nothing that writes in place lies between
        auto held = heldDots_.find(op);
        if (held != heldDots_.end()) { emitDot(op, plan, held->second); return; }
        if (Op* partner = sumPartner(op)) {
          size_t q = pos + 1;
          bool clear = true;
          for (; q < r.ops.size() && r.ops[q].get() != partner; ++q) {
            const std::string& between = r.ops[q]->name;
            if (!isFusibleOp(*r.ops[q]) && between != "dot_general" && between != "dot" && between != "reduce" && between != "convolution") clear = false;
          }
          if (clear && q < r.ops.size() && !emitted_.count(partner) && !heldDots_.count(partner)) { heldDots_[partner] = op; return; }
        }
        emitDot(op, plan);
        return;
      }
      if (n == "convolution") { emitConv(op, plan); return; }
      if (n == "scatter") { emitScatter(op, plan); return; }
      if (n == "sort") { emitSort(op, plan); return; }
      if (n == "dynamic_update_slice") { emitDus(op, plan); return; }
      if (n == "while") { emitWhile(op, plan); return; }
      if (n == "case") { emitCase(op, plan); return; }
      throw CompileError("no lowering for stablehlo." + n);
    }
  }

  // Inside a host-counted loop, the counter-selected slice of a tensor that the loop never writes (xs[i], or slice i of a
  // product taken over the whole sequence ahead of the loop) is a contiguous block whose address the host knows at every
  // iteration: the value becomes a name for that block, and the kernels that read it take the address as an argument
  // instead of loading the counter first and the data after it.
  bool sliceBecomesAlias(Op* op, Region& r) {
    static const bool on = !getenv("MI355X_SLICE_ALIASES") || atoi(getenv("MI355X_SLICE_ALIASES")) != 0;
    Value* x = op->operands[0];
    Value* v = op->result();
    if (!on || loopDepth_ != 1 || ivArgs().empty() || !hasStorage(x) || v->type.numel() == 0 || !r.parent || r.parent->name != "while") return false;
    // never written while the loop runs: defined outside it, or a carry handed on unchanged
    bool invariant = regionOf(x) != &r;
    if (x->argOf == &r) {
      Op* ret = r.terminator();
      invariant = ret && (size_t)x->defIndex < ret->operands.size() && ret->operands[(size_t)x->defIndex] == x;
    }
    if (!invariant || st_[storageOf(x)].aliasOf >= 0) return false;
    const auto& sizes = op->ints("sizes");
    const auto& dims = x->type.dims;
    if (sizes.size() != dims.size()) return false;
    // one contiguous block: unit dims, then at most one partial dim, then whole dims
    int last = -1;
    for (int d = 0; d < (int)dims.size(); ++d) if (sizes[(size_t)d] != dims[(size_t)d]) last = d;
    for (int d = 0; d < last; ++d) if (sizes[(size_t)d] != 1) return false;
    int64_t base = 0;
    std::vector<int64_t> perIter;
    if (!hostSlice(op, stridesOf(x->type), base, perIter) || perIter.empty()) return false;
    const int64_t esz = (int64_t)dtypeSize(v->type.dt);
    for (auto& e : perIter) e *= esz;
    P.ivTables.push_back(std::move(perIter));
    const int sid = newAlias(storageOf(x), 0, (int64_t)v->type.bytes(), (int)P.ivTables.size() - 1);
    bind(v, sid);
    emitted_.insert(op);
    return true;
  }

  // a value that analysis left fused but some consumer needs in memory after all
  void materializeNow(Value* v, Plan& plan) {
    if (hasStorage(v)) return;
    if (!v->def || !isFusibleOp(*v->def)) throw CompileError("internal: cannot materialise " + v->name);
    emitMaterialized(v->def, plan);
  }

  // true when materialising `op` takes a kernel (not a constant-pool entry, an alias or nothing)
  bool takesKernel(Op* op) {
    Value* v = op->result();
    const std::string& n = op->name;
    if (n == "constant") {
      auto& d = *op->attrs.at("value").dense;
      if (!d.splat || d.type.numel() == 1) return false;
    }
    if ((n == "reshape" || isPassThrough(*op) || (n == "convert" && op->operands[0]->type.dt == v->type.dt)) && hasStorage(op->operands[0])) return false;
    return v->type.numel() != 0;
  }

  // Values the loop kernel of `v` would read, given that `roots` are computed in the same kernel.
  // Returns false when one of them is not in memory yet.
  bool leavesReady(Value* v, const std::vector<Value*>& roots, std::unordered_set<Value*>& seen, int& count) {
    for (auto* o : v->def->operands) {
      if (!seen.insert(o).second) continue;
      if (std::find(roots.begin(), roots.end(), o) != roots.end()) {
        // a value that must live in memory (it is read at shifted positions) cannot feed a kernel that also computes it
        if (o->def && o->def->has("force_materialize")) return false;
        continue;
      }
      if (hasStorage(o)) { ++count; continue; }
      if (!o->def || !isFusibleOp(*o->def) || o->def->results.size() != 1 || needMat_[o]) return false;
      if (!leavesReady(o, roots, seen, count)) return false;
    }
    return true;
  }

  // Materialised elementwise values with the same dims whose inputs are already in memory are
  // computed by one kernel with several outputs: later ops of the region are pulled forward
  // (SSA values are pure, so computing them earlier is always valid).
  // A large elementwise value whose first reader is a column-style reduction over the same index space (the masked
  // gradient that batch norm's backward pass sums twice before it uses it element by element): the reduction's pass
  // over the data computes it anyway, visits every element exactly once and can store it, so the value needs no
  // kernel of its own and the reduction does not read it back.  True when `op`'s result is such a value and nothing
  // before that reduction needs it in memory.
  bool storedByAReduction(Op* op, Region& r, size_t pos) {
    static const bool on = !getenv("MI355X_REDUCE_STORES") || atoi(getenv("MI355X_REDUCE_STORES")) != 0;
    Value* v = op->result();
    // (a reduction over a small input is one launch of a few workgroups: too few to also compute and store the value)
    // (a one-pass reduction over a small input still has a few dozen workgroups, see the column tiles in codegen.cc, and the
    // launch saved is worth more than they are; below 16 384 elements the value is cheaper to recompute than to wait for)
    const bool sized = v->type.numel() >= 16384;
    if (!on || !sized || !takesKernel(op) || op->name == "constant" || op->has("force_materialize")) return false;
    if (v->type.dt != DType::F32 && v->type.dt != DType::BF16) return false;
    Op* red = nullptr;
    size_t posRed = 0;
    for (size_t q = pos + 1; q < r.ops.size() && q <= pos + 48 && !red; ++q) {
      Op* y = r.ops[q].get();
      if (y->name != "reduce" || emitted_.count(y) || !isSimpleReduce(*y)) continue;
      if (y->operands[0]->type.dims != v->type.dims || !reduceIsColumnStyle(y)) continue;
      std::vector<Value*> leaves;
      std::unordered_set<Value*> seen;
      collectLeavesOf(y->operands[0], leaves, seen);
      if (std::find(leaves.begin(), leaves.end(), v) != leaves.end()) { red = y; posRed = q; }
    }
    if (!red) return false;
    // every reader of the value that comes before the reduction must be content with recomputing it (none should: it
    // would not have been marked for memory otherwise), and readers in nested regions need it in memory at once
    for (Op* u : v->users) {
      if (u->parent != &r) return false;
      size_t pu = 0;
      while (pu < r.ops.size() && r.ops[pu].get() != u) ++pu;
      if (pu < posRed && (!isFusibleOp(*u) || needMat_[u->result()])) return false;
    }
    // what the value is computed from must be in memory by now
    std::vector<Value*> mine;
    std::unordered_set<Value*> seen;
    for (auto* o : op->operands) collectLeavesOf(o, mine, seen);
    for (auto* l : mine) if (!hasStorage(l)) return false;
    return true;
  }

  void emitLoopGroup(Op* op, Region& r, size_t pos, Plan& plan) {
    Value* v = op->result();
    static const bool multi = !(getenv("MI355X_MULTI_OUTPUT") && getenv("MI355X_MULTI_OUTPUT")[0] == '0');
    if (hasStorage(v)) return;
    if (!multi || !takesKernel(op)) { emitMaterialized(op, plan); return; }
    std::vector<Value*> roots{v};
    std::vector<Op*> members{op};
    std::unordered_set<Value*> seen;
    int leafCount = 0;
    leavesReady(v, roots, seen, leafCount);
    const size_t kLookAhead = 96, kMaxRoots = 8;
    for (size_t q = pos + 1; q < r.ops.size() && q <= pos + kLookAhead && roots.size() < kMaxRoots; ++q) {
      Op* y = r.ops[q].get();
      if (emitted_.count(y) || !isFusibleOp(*y) || y->results.size() != 1) continue;
      Value* w = y->result();
      if (!needMat_[w] || hasStorage(w)) continue;
      if (w->type.dims != v->type.dims || dtypeSize(w->type.dt) != dtypeSize(v->type.dt)) continue;
      if (!takesKernel(y)) continue;
      std::unordered_set<Value*> seenY = seen;
      int cnt = leafCount;
      if (!leavesReady(w, roots, seenY, cnt) || cnt + (int)roots.size() + 1 > 40) continue;
      seen = std::move(seenY);
      leafCount = cnt;
      roots.push_back(w);
      members.push_back(y);
    }
    if (roots.size() == 1) { emitMaterialized(op, plan); return; }
    FusedCode fc = generateLoopKernel(roots, leafPred());
    std::string label = "fusion:" + op->name;
    for (size_t k = 1; k < members.size(); ++k) label += "+" + members[k]->name;
    for (auto* w : roots) bind(w, newStorage(w->type.bytes()));
    for (auto* m : members) emitted_.insert(m);
    addFused(plan, fc, label + " " + v->type.str(), roots);
  }

  void emitMaterialized(Op* op, Plan& plan) {
    Value* v = op->result();
    if (hasStorage(v)) return;
    const std::string& n = op->name;
    if (n == "constant") {
      auto& d = *op->attrs.at("value").dense;
      if (!d.splat || d.type.numel() == 1) {
        int64_t off = ((int64_t)P.constPool.size() + kAlign - 1) / kAlign * kAlign;
        P.constPool.resize((size_t)off + std::max<size_t>(d.bytes.size(), 4));
        memcpy(P.constPool.data() + off, d.bytes.data(), d.bytes.size());
        int sid = newStorage(d.bytes.size(), BufRef::Const);
        st_[sid].offset = off;
        bind(v, sid);
        return;
      }
    }
    if ((n == "reshape" || isPassThrough(*op) || (n == "convert" && op->operands[0]->type.dt == v->type.dt)) && hasStorage(op->operands[0])) {
      bind(v, storageOf(op->operands[0]));
      return;
    }
    if (v->type.numel() == 0) {
      bind(v, newStorage(4));
      return;
    }
    FusedCode fc = generateLoopKernel(v, leafPred());
    int sid = newStorage(v->type.bytes());
    bind(v, sid);
    addFused(plan, fc, "fusion:" + n + " " + v->type.str(), {v});
  }

  void collectLeavesOf(Value* v, std::vector<Value*>& out, std::unordered_set<Value*>& seen) {
    if (!seen.insert(v).second) return;
    if (hasStorage(v)) { out.push_back(v); return; }
    if (!v->def || !isFusibleOp(*v->def) || needMat_[v]) { out.push_back(v); return; }
    for (auto* o : v->def->operands) collectLeavesOf(o, out, seen);
  }

  // Softmax / LayerNorm shaped subgraphs: reductions over the trailing dims, elementwise values
  // that read them back through a broadcast, possibly further reductions of those, all computed
  // in one kernel that owns whole rows (reference: the mps.softmax / mps.layer_norm custom calls
  // its fusion passes produce, passes/fuse_softmax.cc:174-247, passes/fuse_layer_norm.cc:229-354).
  bool tryRowProgram(Op* op, Region& r, size_t pos, Plan& plan) {
    static const bool enabled = !(getenv("MI355X_ROW_PROGRAMS") && getenv("MI355X_ROW_PROGRAMS")[0] == '0');
    if (!enabled || !isSimpleReduce(*op)) return false;
    const TensorType& xt = op->operands[0]->type;
    std::vector<int64_t> rd = op->ints("dimensions");
    std::sort(rd.begin(), rd.end());
    int rank = xt.rank();
    if (rd.empty() || (int)rd.size() >= rank) return false;
    for (size_t q = 0; q < rd.size(); ++q) if (rd[q] != rank - (int)rd.size() + (int)q) return false;
    std::vector<int64_t> keptShape(xt.dims.begin(), xt.dims.end() - rd.size());
    int64_t Kn = 1, Rn = 1;
    for (auto d : keptShape) Kn *= d;
    for (size_t q = keptShape.size(); q < xt.dims.size(); ++q) Rn *= xt.dims[q];
    if (Kn < 256 || Rn < 2 || Rn > 32768) return false;

    RowProgram rp;
    std::unordered_map<Value*, int> phaseOf;
    std::unordered_set<Op*> inlined;      // fusible ops evaluated inside the kernel
    std::vector<Op*> rootOps, candidates;
    std::vector<std::vector<Op*>> candidateDeps;
    // can `v` be evaluated in the kernel?  dep = 1 + the latest phase it needs
    std::function<bool(Value*, int&, std::vector<Op*>&)> can = [&](Value* v, int& dep, std::vector<Op*>& seen) -> bool {
      if (hasStorage(v)) return true;
      auto ph = phaseOf.find(v);
      if (ph != phaseOf.end()) { dep = std::max(dep, ph->second + 1); return true; }
      Op* d = v->def;
      if (!d || !isFusibleOp(*d) || d->results.size() != 1 || d->parent != &r) return false;
      if (std::find(seen.begin(), seen.end(), d) != seen.end()) return true;
      seen.push_back(d);
      if (seen.size() > 256) return false;
      for (auto* o : d->operands) if (!can(o, dep, seen)) return false;
      return true;
    };
    const size_t kWindow = 96;
    for (size_t q = pos; q < r.ops.size() && q <= pos + kWindow; ++q) {
      Op* y = r.ops[q].get();
      if (emitted_.count(y)) continue;
      if (y->name == "reduce") {
        if (!isSimpleReduce(*y) || y->operands[0]->type.dims != xt.dims) { if (y == op) return false; continue; }
        std::vector<int64_t> yd = y->ints("dimensions");
        std::sort(yd.begin(), yd.end());
        if (yd != rd) continue;
        int dep = 0;
        std::vector<Op*> seen;
        if (!can(y->operands[0], dep, seen) || !can(y->operands[1], dep, seen)) { if (y == op) return false; continue; }
        if (dep > (int)rp.phases.size()) continue;
        if (dep == (int)rp.phases.size()) rp.phases.emplace_back();
        if (rp.phases[dep].size() >= 4) continue;
        rp.phases[dep].push_back(y);
        phaseOf[y->result()] = dep;
        for (auto* z : seen) inlined.insert(z);
        continue;
      }
      if (rp.phases.empty()) return false;
      if (!isFusibleOp(*y) || y->results.size() != 1) continue;
      Value* w = y->result();
      if (!needMat_[w] || hasStorage(w) || !takesKernel(y)) continue;
      if (w->type.dims != xt.dims && w->type.dims != keptShape) continue;
      int dep = 0;
      std::vector<Op*> seen;
      if (!can(w, dep, seen) || dep == 0) continue;
      candidates.push_back(y);
      candidateDeps.push_back(std::move(seen));
    }
    if (rp.phases.empty() || rp.phases[0].empty() || rp.phases[0][0] != op) return false;
    // Candidates in reverse program order: one whose readers are all inside the kernel is not
    // stored (it is recomputed where needed); the others become outputs.
    std::unordered_set<Op*> members(inlined.begin(), inlined.end());
    for (auto& ph : rp.phases) for (auto* y : ph) members.insert(y);
    std::vector<Op*> dropped;
    for (int c = (int)candidates.size() - 1; c >= 0; --c) {
      Op* y = candidates[c];
      Value* w = y->result();
      bool inside = !w->users.empty();
      for (Op* u : w->users) if (!members.count(u)) inside = false;
      if (inside) continue;   // stays an inlined intermediate if a member reads it, otherwise untouched
      if (rp.fullRoots.size() + rp.keptRoots.size() >= 8) continue;
      (w->type.dims == xt.dims ? rp.fullRoots : rp.keptRoots).push_back(w);
      rootOps.push_back(y);
      members.insert(y);
      for (auto* z : candidateDeps[c]) { inlined.insert(z); members.insert(z); }
    }
    if (rp.phases.size() == 1 && rp.fullRoots.empty()) return false;   // plain reductions: the partial-sum kernels do better
    // inlined values that were going to be written to memory: dropped when every reader is in the kernel
    for (auto* z : inlined) {
      Value* w = z->result();
      if (!needMat_[w] || hasStorage(w)) continue;
      if (std::find(rootOps.begin(), rootOps.end(), z) != rootOps.end()) continue;
      bool inside = true;
      for (Op* u : w->users) if (!members.count(u)) inside = false;
      if (inside) { dropped.push_back(z); continue; }
      bool full = w->type.dims == xt.dims, kept = w->type.dims == keptShape;
      if ((!full && !kept) || !takesKernel(z) || rp.fullRoots.size() + rp.keptRoots.size() >= 10) return false;
      (full ? rp.fullRoots : rp.keptRoots).push_back(w);
      rootOps.push_back(z);
    }
    FusedCode fc;
    try {
      fc = generateRowProgram(rp, leafPred());
    } catch (const CompileError&) {
      return false;
    }
    std::vector<Value*> outs;
    std::string label = "rows:";
    for (auto& ph : rp.phases) {
      for (auto* y : ph) {
        bind(y->result(), newStorage(y->result()->type.bytes()));
        outs.push_back(y->result());
        emitted_.insert(y);
        label += "reduce,";
      }
      label += "|";
    }
    for (auto* y : rootOps) {
      bind(y->result(), newStorage(y->result()->type.bytes()));
      outs.push_back(y->result());
      emitted_.insert(y);
      label += y->name + ",";
    }
    for (auto* z : dropped) emitted_.insert(z);
    addFused(plan, fc, label + " " + xt.str(), outs);
    return true;
  }

  void emitRegionReduce(Op* op, Plan& plan) {
    size_t n = op->operands.size() / 2;
    for (size_t j = 0; j < n; ++j) {
      // init values must be readable
      std::vector<Value*> il;
      std::unordered_set<Value*> seen;
      collectLeavesOf(op->operands[n + j], il, seen);
      for (auto* l : il) if (!hasStorage(l)) materializeNow(l, plan);
    }
    std::vector<Value*> outs;
    for (auto& r : op->results) outs.push_back(r.get());
    if (outs.empty() || outs[0]->type.numel() == 0) {
      for (auto* o : outs) bind(o, newStorage(4));
      return;
    }
    if (op->operands[0]->type.numel() == 0) throw CompileError("stablehlo.reduce over an empty tensor is not supported");
    FusedCode fc = generateRegionReduce(op, leafPred());
    for (auto* o : outs) bind(o, newStorage(o->type.bytes()));
    emitted_.insert(op);
    addFused(plan, fc, "reduce(region) " + op->operands[0]->type.str() + " -> " + outs[0]->type.str(), outs);
  }

  void emitReduce(Op* op, Region& r, Plan& plan) {
    if (!isSimpleReduce(*op)) { emitRegionReduce(op, plan); return; }
    std::vector<Op*> group{op};
    std::vector<Value*> myLeaves;
    {
      std::unordered_set<Value*> seen;
      collectLeavesOf(op->operands[0], myLeaves, seen);
    }
    // values held back for this reduction to store (storedByAReduction); any that it cannot take get their own kernel now
    std::vector<Value*> side;
    const bool columnStyle = reduceIsColumnStyle(op);
    auto takeSide = [&](Value* l) {
      if (!deferred_.count(l) || hasStorage(l)) return false;
      if (std::find(side.begin(), side.end(), l) != side.end()) return true;
      if (columnStyle && side.size() < 2 && l->type.dims == op->operands[0]->type.dims) { side.push_back(l); return true; }
      materializeNow(l, plan);
      return false;
    };
    for (auto* l : myLeaves) takeSide(l);
    // sibling reductions over the same index space that share an input: one pass over memory
    bool seenSelf = false;
    for (auto& qp : r.ops) {
      Op* q = qp.get();
      if (q == op) { seenSelf = true; continue; }
      if (!seenSelf || group.size() >= 4) continue;
      if (q->name != "reduce" || emitted_.count(q) || !isSimpleReduce(*q)) continue;
      if (q->operands[0]->type.dims != op->operands[0]->type.dims) continue;
      auto a = q->ints("dimensions"), b = op->ints("dimensions");
      std::sort(a.begin(), a.end());
      std::sort(b.begin(), b.end());
      if (a != b) continue;
      std::vector<Value*> ql;
      std::unordered_set<Value*> seen;
      collectLeavesOf(q->operands[0], ql, seen);
      collectLeavesOf(q->operands[1], ql, seen);
      bool ready = true, shares = false;
      for (auto* l : ql) {
        if (!hasStorage(l) && !takeSide(l)) ready = hasStorage(l);
        if (std::find(myLeaves.begin(), myLeaves.end(), l) != myLeaves.end() && l->type.numel() > kSmallNumel) shares = true;
      }
      if (ready && shares) group.push_back(q);
    }
    for (auto* g : group) {
      // the init value must be readable
      std::vector<Value*> il;
      std::unordered_set<Value*> seen;
      collectLeavesOf(g->operands[1], il, seen);
      for (auto* l : il) if (!hasStorage(l)) materializeNow(l, plan);
    }
    if (op->result()->type.numel() == 0) {
      for (auto* g : group) { bind(g->result(), newStorage(4)); emitted_.insert(g); }
      return;
    }
    if (op->operands[0]->type.numel() == 0) {
      // reducing nothing: the result is the init value broadcast
      throw CompileError("stablehlo.reduce over an empty tensor is not supported");
    }
    // Per-output values that need nothing but the results and inputs of the result shape (a mean, a
    // variance, a reciprocal square root ...) ride along in the pass that folds the partial sums.
    std::vector<Value*> epilogue;
    std::vector<Op*> epilogueOps;
    {
      std::unordered_set<Value*> results;
      for (auto* g : group) results.insert(g->result());
      const auto& keptDims = op->result()->type.dims;
      std::unordered_set<Value*> counted;
      std::function<bool(Value*, bool&, int&)> can = [&](Value* v, bool& usesResult, int& budget) -> bool {
        if (results.count(v) || std::find(epilogue.begin(), epilogue.end(), v) != epilogue.end()) { usesResult = true; return true; }
        if (hasStorage(v)) return v->type.numel() <= op->result()->type.numel();   // nothing bigger than the result shape
        Op* d = v->def;
        if (!d || !isFusibleOp(*d) || d->results.size() != 1 || d->parent != &r || needMat_[v]) return false;
        if (!counted.insert(v).second) return true;   // a shared subexpression is generated once
        if (--budget < 0) return false;
        // the lane that holds a finished result knows that one only: whatever stands between the result and the value
        // must read it where it is evaluated itself (a slice, a reversal or a concatenation reads another output's)
        for (auto* o : d->operands) {
          bool below = false;
          if (!can(o, below, budget)) return false;
          if (below && (movesData(*d) || o->type.dims != v->type.dims)) return false;
          usesResult |= below;
        }
        return true;
      };
      size_t pos = 0;
      while (pos < r.ops.size() && r.ops[pos].get() != op) ++pos;
      for (size_t q = pos + 1; q < r.ops.size() && q <= pos + 512 && epilogue.size() < 6; ++q) {
        Op* y = r.ops[q].get();
        if (emitted_.count(y) || !isFusibleOp(*y) || y->results.size() != 1) continue;
        Value* w = y->result();
        if (!needMat_[w] || hasStorage(w) || !takesKernel(y) || w->type.dims != keptDims) continue;
        bool uses = false;
        int budget = 64;
        bool ok = true;
        counted.clear();
        for (auto* o : y->operands) {
          bool below = false;
          if (!can(o, below, budget) || (below && (movesData(*y) || o->type.dims != keptDims))) ok = false;
          uses |= below;
        }
        if (!ok || !uses) continue;
        epilogue.push_back(w);
        epilogueOps.push_back(y);
      }
    }
    // Batch-norm statistics of a convolution's output: when the step just emitted is the convolution that produced the
    // reduced tensor, the reductions are its column sum and column sum of squares, and the kernel can take them from
    // its accumulators (per tile row), the pass over the output is dropped and only the fold of the tile rows remains.
    int64_t statRows = 0;
    int sumAt = -1, sqAt = -1;
    static const bool statsOn = !getenv("MI355X_CONV_STATS") || atoi(getenv("MI355X_CONV_STATS")) != 0;
    if (statsOn && group.size() == 2 && !plan.steps.empty() && plan.steps.back().kind == Step::Conv && plan.steps.back().statsArg < 0) {
      Step& cs = plan.steps.back();
      Value* y = nullptr;
      Value* ySquared = nullptr;
      for (int j = 0; j < 2; ++j) {
        Value* x = group[(size_t)j]->operands[0];
        const char* kind = simpleReduceKind(*group[(size_t)j]);
        if (!kind || std::string(kind) != "add") { sumAt = sqAt = -2; break; }
        if (hasStorage(x)) { sumAt = sumAt == -1 ? j : -2; y = x; }
        else if (x->def && x->def->name == "multiply" && x->def->operands[0] == x->def->operands[1] && hasStorage(x->def->operands[0])) { sqAt = sqAt == -1 ? j : -2; ySquared = x->def->operands[0]; }
      }
      bool ok = sumAt >= 0 && sqAt >= 0 && y == ySquared && y->type.dt == DType::F32 && cs.args.size() >= 3 && cs.args[2].index == storageOf(y) && cs.conv.type == DType::F32;
      if (ok) {
        // every dim but the last (the feature axis) is reduced
        auto dims = op->ints("dimensions");
        std::sort(dims.begin(), dims.end());
        ok = (int)dims.size() == y->type.rank() - 1;
        for (size_t k = 0; ok && k < dims.size(); ++k) ok = dims[k] == (int64_t)k;
      }
      if (ok) {
        mi355_conv_desc abi = toAbi(cs.conv);
        statRows = mi355_conv_stats_rows(&abi);
        if (statRows > 0 && (int64_t)abi.O != y->type.dims.back()) statRows = 0;
      }
    }
    if (statRows > 0 && !side.empty()) {   // (the folding pass of convolution statistics walks no data)
      for (auto* l : side) materializeNow(l, plan);
      side.clear();
    }
    FusedCode fc = generateReduceKernel(group, leafPred(), epilogue, statRows, side);
    if (!side.empty() && !fc.sideStored) {
      for (auto* l : side) materializeNow(l, plan);
      side.clear();
      fc = generateReduceKernel(group, leafPred(), epilogue, statRows);
    }
    std::vector<Value*> outs;
    for (auto* g : group) {
      bind(g->result(), newStorage(g->result()->type.bytes()));
      outs.push_back(g->result());
      emitted_.insert(g);
    }
    std::string label = (group.size() > 1 ? "reduce x" + std::to_string(group.size()) : std::string("reduce"));
    if (statRows > 0) label = "fold of convolution statistics, " + label;
    if (fc.epilogueFused) {
      for (size_t k = 0; k < epilogue.size(); ++k) {
        bind(epilogue[k], newStorage(epilogue[k]->type.bytes()));
        outs.push_back(epilogue[k]);
        emitted_.insert(epilogueOps[k]);
        label += "+" + epilogueOps[k]->name;
      }
    }
    for (auto* l : side) {
      bind(l, newStorage(l->type.bytes()));
      outs.push_back(l);
      emitted_.insert(l->def);
      label += " storing " + l->def->name;
    }
    if (statRows > 0) {
      ProducerStats ps;
      ps.step = plan.steps.size() - 1;
      ps.sumOffset = fc.partialOffsets[(size_t)sumAt];
      ps.sqOffset = fc.partialOffsets[(size_t)sqAt];
      addFused(plan, fc, label + " " + group[0]->operands[0]->type.str() + " -> " + outs[0]->type.str(), outs, &ps);
    } else {
      addFused(plan, fc, label + " " + group[0]->operands[0]->type.str() + " -> " + outs[0]->type.str(), outs);
    }
  }

  static std::vector<int64_t> stridesOf(const TensorType& t) {
    std::vector<int64_t> s(t.rank(), 1);
    for (int d = t.rank() - 2; d >= 0; --d) s[d] = s[d + 1] * t.dims[d + 1];
    return s;
  }

  // merge an ordered list of dims into (size, stride); false if they do not collapse
  static bool mergeDims(const TensorType& t, const std::vector<int64_t>& dims, int64_t& size, int64_t& stride) {
    return mergeDims(t, stridesOf(t), dims, size, stride);
  }
  static bool mergeDims(const TensorType& t, const std::vector<int64_t>& st, const std::vector<int64_t>& dims, int64_t& size, int64_t& stride) {
    size = 1;
    stride = 0;
    bool have = false;
    int64_t expect = 0;
    for (size_t k = 0; k < dims.size(); ++k) {
      int64_t d = dims[k];
      if (t.dims[d] == 1) continue;
      if (!have) { have = true; size = t.dims[d]; stride = st[d]; expect = st[d]; continue; }
      // dims are listed outer to inner: the next one must tile the previous stride exactly
      if (st[d] * t.dims[d] != expect) return false;
      size *= t.dims[d];
      stride = st[d];
      expect = st[d];
    }
    if (!have) stride = 1;
    return true;
  }

  // ---------------------------------------------------------------- strided views
  // A dot_general operand that is a slice / reshape / transpose chain over a buffer is read through
  // element strides and a base offset instead of being copied out first (the split of a fused QKV
  // projection into heads is such a chain).
  struct View {
    Value* root = nullptr;          // value that owns the memory
    int64_t offset = 0;             // elements from the root's first element
    std::vector<int64_t> strides;   // per dim of the viewed value
    std::vector<int64_t> iterOffsets;   // inside a host-counted loop: further elements at iteration k (a slice taken at the counter)
  };

  // ---------------------------------------------------------------- loop counters the host follows
  // The counter carry of a counted loop (init constant, constant step, static trip count) takes known values, so
  // nothing needs to compute it on the device: kernels read entry k of a table of its values at iteration k, and a
  // dynamic_slice whose start indices are scalar integer arithmetic on the counter is a view whose offset the host
  // computes per iteration.  That removes the counter's own kernel from every iteration and lets products read
  // xs[i] in place (the reference re-evaluates such slices on the device every iteration: ops/control_flow.cc:702-989).
  struct IvInfo { int64_t init = 0, step = 0, trip = 0; };
  static std::unordered_map<const Value*, IvInfo>& ivArgs() {
    static thread_local std::unordered_map<const Value*, IvInfo> m;
    return m;
  }

  // value of the scalar integer `v` at iteration k of the host-counted loop it depends on (if any); `trip` receives that
  // loop's trip count (0 when `v` is a plain constant)
  static bool evalIndex(Value* v, int64_t k, int64_t& out, int64_t& trip, int depth = 0) {
    if (depth > 16 || v->type.numel() != 1) return false;
    auto it = ivArgs().find(v);
    if (it != ivArgs().end()) {
      if (trip != 0 && trip != it->second.trip) return false;
      trip = it->second.trip;
      out = it->second.init + k * it->second.step;
      return true;
    }
    if (constInt(v, out)) return true;
    Op* d = v->def;
    if (!d || d->results.size() != 1 || !(isInt(v->type.dt) || v->type.dt == DType::Pred)) return false;
    std::vector<int64_t> in;
    for (auto* o : d->operands) {
      int64_t x;
      if (!evalIndex(o, k, x, trip, depth + 1)) return false;
      in.push_back(x);
    }
    const std::string& n = d->name;
    auto wrap = [&](int64_t x) {   // two's complement of the value's own width
      const size_t sz = dtypeSize(v->type.dt);
      if (v->type.dt == DType::Pred) return (int64_t)(x != 0);
      if (sz >= 8) return x;
      const int bits = (int)(8 * sz);
      uint64_t u = (uint64_t)x & ((1ull << bits) - 1);
      if (isSignedInt(v->type.dt) && (u >> (bits - 1))) return (int64_t)(u | ~((1ull << bits) - 1));
      return (int64_t)u;
    };
    if (n == "reshape" || n == "convert" || n == "broadcast_in_dim") { out = wrap(in[0]); return true; }
    if (in.size() == 1 && n == "negate") { out = wrap(-in[0]); return true; }
    if (in.size() == 2) {
      if (n == "add") { out = wrap(in[0] + in[1]); return true; }
      if (n == "subtract") { out = wrap(in[0] - in[1]); return true; }
      if (n == "multiply") { out = wrap(in[0] * in[1]); return true; }
      if (n == "minimum") { out = std::min(in[0], in[1]); return true; }
      if (n == "maximum") { out = std::max(in[0], in[1]); return true; }
      if (n == "compare" && isSignedInt(d->operands[0]->type.dt)) {
        const std::string& dir = d->str("direction");
        out = dir == "LT" ? in[0] < in[1] : dir == "LE" ? in[0] <= in[1] : dir == "GT" ? in[0] > in[1] : dir == "GE" ? in[0] >= in[1] : dir == "EQ" ? in[0] == in[1] : in[0] != in[1];
        return true;
      }
    }
    if (in.size() == 3 && n == "select") { out = in[0] ? in[1] : in[2]; return true; }
    if (in.size() == 3 && n == "clamp") { out = std::min(std::max(in[1], in[0]), in[2]); return true; }
    return false;
  }

  // a dynamic_slice all of whose start indices the host can evaluate; `perIter` receives the element offset at each
  // iteration relative to `strides` (empty when every index is a constant), `base` the constant part
  static bool hostSlice(const Op* d, const std::vector<int64_t>& strides, int64_t& base, std::vector<int64_t>& perIter) {
    if (!d || d->name != "dynamic_slice") return false;
    const TensorType& xt = d->operands[0]->type;
    auto& sizes = d->ints("sizes");
    if ((int)d->operands.size() != 1 + xt.rank() || (int)sizes.size() != xt.rank()) return false;
    int64_t trip = 0;
    for (int dim = 0; dim < xt.rank(); ++dim) {
      int64_t x;
      if (!evalIndex(d->operands[(size_t)dim + 1], 0, x, trip)) return false;
    }
    const int64_t iters = std::max<int64_t>(trip, 1);
    std::vector<int64_t> offs((size_t)iters, 0);
    for (int64_t k = 0; k < iters; ++k) {
      for (int dim = 0; dim < xt.rank(); ++dim) {
        int64_t x = 0, t2 = 0;
        if (!evalIndex(d->operands[(size_t)dim + 1], k, x, t2)) return false;
        x = std::min(std::max<int64_t>(x, 0), xt.dims[(size_t)dim] - sizes[(size_t)dim]);   // start indices are clamped into range
        offs[(size_t)k] += x * strides[(size_t)dim];
      }
    }
    base = 0;
    perIter.clear();
    if (trip == 0) base = offs[0];
    else perIter = offs;
    return true;
  }

  // strides of `newDims` over memory laid out as (oldDims, oldStrides), if no copy is needed
  static bool reshapeStrides(const std::vector<int64_t>& oldDims, const std::vector<int64_t>& oldStrides, const std::vector<int64_t>& newDims,
                             std::vector<int64_t>& out) {
    std::vector<int64_t> od, os;
    for (size_t i = 0; i < oldDims.size(); ++i) if (oldDims[i] != 1) { od.push_back(oldDims[i]); os.push_back(oldStrides[i]); }
    out.assign(newDims.size(), 0);
    size_t oi = 0, ni = 0;
    while (ni < newDims.size()) {
      if (newDims[ni] == 1) { out[ni++] = 0; continue; }
      if (oi >= od.size()) return false;
      // grow a group of old dims and a group of new dims until their sizes agree
      size_t o0 = oi, n0 = ni;
      int64_t op = od[oi++], np = newDims[ni++];
      while (op != np) {
        if (op < np) { if (oi >= od.size()) return false; op *= od[oi++]; }
        else {
          while (ni < newDims.size() && newDims[ni] == 1) out[ni++] = 0;
          if (ni >= newDims.size()) return false;
          np *= newDims[ni++];
        }
      }
      // the old group must itself be contiguous in its own strides
      for (size_t k = o0; k + 1 < oi; ++k) if (os[k] != os[k + 1] * od[k + 1]) return false;
      int64_t st = os[oi - 1];
      for (size_t k = ni; k-- > n0;) {
        if (newDims[k] == 1) { out[k] = 0; continue; }
        out[k] = st;
        st *= newDims[k];
      }
    }
    return oi == od.size();
  }

  static bool isViewOp(const Op* d) {
    if (!d || d->results.size() != 1) return false;
    if (d->name == "reshape" || d->name == "slice" || d->name == "transpose") return true;
    int64_t base;
    std::vector<int64_t> perIter;
    return d->name == "dynamic_slice" && hostSlice(d, stridesOf(d->operands[0]->type), base, perIter);
  }

  // `ownsMemory(v)`: the caller's notion of "v is (or will be) in memory".
  template <typename F>
  static bool resolveView(Value* v, const F& ownsMemory, View& out) {
    if (ownsMemory(v)) {
      out.root = v;
      out.offset = 0;
      out.strides = stridesOf(v->type);
      return true;
    }
    Op* d = v->def;
    if (!isViewOp(d) || v->type.numel() == 0) return false;
    View in;
    if (!resolveView(d->operands[0], ownsMemory, in)) return false;
    const TensorType& xt = d->operands[0]->type;
    out.root = in.root;
    out.offset = in.offset;
    out.iterOffsets = in.iterOffsets;
    if (d->name == "dynamic_slice") {
      int64_t base = 0;
      std::vector<int64_t> perIter;
      if (!hostSlice(d, in.strides, base, perIter)) return false;
      out.offset += base;
      out.strides = in.strides;
      if (!perIter.empty()) {
        if (out.iterOffsets.empty()) out.iterOffsets = perIter;
        else if (out.iterOffsets.size() == perIter.size()) for (size_t k = 0; k < perIter.size(); ++k) out.iterOffsets[k] += perIter[k];
        else return false;
      }
      return true;
    }
    if (d->name == "slice") {
      auto& start = d->ints("start");
      auto& stride = d->ints("strides");
      out.strides.resize(xt.rank());
      for (int k = 0; k < xt.rank(); ++k) {
        out.offset += start[k] * in.strides[k];
        out.strides[k] = in.strides[k] * (stride.empty() ? 1 : stride[k]);
      }
      return true;
    }
    if (d->name == "transpose") {
      auto& perm = d->ints("dims");
      out.strides.resize(perm.size());
      for (size_t k = 0; k < perm.size(); ++k) out.strides[k] = in.strides[perm[k]];
      return true;
    }
    return reshapeStrides(xt.dims, in.strides, v->type.dims, out.strides);
  }

  // values that are in memory whatever the fusion analysis decides: arguments, results of ops that
  // are steps of their own, and bias sums folded into their product
  static bool alwaysInMemory(Value* v) {
    if (!v->def) return true;
    if (!isFusibleOp(*v->def)) return v->def->name != "return";
    // the sum a product step may write itself (with its bias, with an addend, with a second product): the bare product
    // is then never stored, so the sum cannot be recomputed from it
    if (v->def->name == "add")
      for (auto* o : v->def->operands)
        if (o->def && (o->def->name == "dot_general" || o->def->name == "dot") && o->users.size() == 1) return true;
    return false;
  }

  static bool dotTakesView(Value* v, Op* user) {
    static const bool views = !getenv("MI355X_GEMM_VIEWS") || atoi(getenv("MI355X_GEMM_VIEWS")) != 0;
    if (!views || (user->name != "dot_general" && user->name != "dot") || !isViewOp(v->def)) return false;
    if (v->type.dt != DType::F32 && v->type.dt != DType::BF16) return false;
    View vw;
    return resolveView(v, alwaysInMemory, vw);
  }


  // ---------------------------------------------------------------- activation epilogue of a product
  // The elementwise chain that follows a bf16 product (after its bias) is recognised by what it computes, not by
  // how it is written: the chain is evaluated on the host at a handful of points as a function of the one value
  // it reads, and accepted when y = a x (1 + tanh(c (x + b x^3))) fits, with a, b, c read off the evaluations
  // (the tanh form of GELU; jax.nn.gelu(approximate=True) and hand-written variants associate the products
  // differently and carry their constants in the tensor's own precision).
  struct ActMatch {
    Value* out = nullptr;
    std::vector<Op*> ops;
    float a = 0.f, b = 0.f, c = 0.f;
  };

  static bool splatNumber(Op* cst, double& out) {
    auto& dd = *cst->attrs.at("value").dense;
    if (!dd.splat && dd.type.numel() != 1) return false;
    const uint8_t* p = dd.bytes.data();
    switch (dd.type.dt) {
      case DType::F32: { float f; memcpy(&f, p, 4); out = f; return true; }
      case DType::BF16: { uint16_t h; memcpy(&h, p, 2); uint32_t u = (uint32_t)h << 16; float f; memcpy(&f, &u, 4); out = f; return true; }
      case DType::F16: { _Float16 h; memcpy(&h, p, 2); out = (double)h; return true; }
      case DType::S32: { int32_t i; memcpy(&i, p, 4); out = i; return true; }
      default: return false;
    }
  }

  // value of `v` when `x` holds `at`; false when the chain leaves the ops a scalar evaluation covers
  static bool evalChain(Value* v, Value* x, double at, std::unordered_map<Value*, double>& memo, double& out) {
    if (v == x) { out = at; return true; }
    auto it = memo.find(v);
    if (it != memo.end()) { out = it->second; return true; }
    Op* d = v->def;
    if (!d || d->results.size() != 1) return false;
    const std::string& n = d->name;
    double a = 0, b = 0;
    bool ok = true;
    if (n == "constant") ok = splatNumber(d, out);
    else if (n == "broadcast_in_dim" || n == "reshape" || n == "convert") ok = evalChain(d->operands[0], x, at, memo, out);
    else if (n == "add" || n == "subtract" || n == "multiply" || n == "divide" || n == "power") {
      ok = evalChain(d->operands[0], x, at, memo, a) && evalChain(d->operands[1], x, at, memo, b);
      out = n == "add" ? a + b : n == "subtract" ? a - b : n == "multiply" ? a * b : n == "divide" ? a / b : std::pow(a, b);
    } else if (n == "tanh" || n == "negate" || n == "exponential" || n == "logistic") {
      ok = evalChain(d->operands[0], x, at, memo, a);
      out = n == "tanh" ? std::tanh(a) : n == "negate" ? -a : n == "exponential" ? std::exp(a) : 1.0 / (1.0 + std::exp(-a));
    } else ok = false;
    if (ok) memo[v] = out;
    return ok;
  }

  // the chain of same-shape elementwise ops that is the only reader of `x` and has one value read from outside
  bool matchActivation(Value* x, ActMatch& m) {
    const bool on = !strictBf16() && (!getenv("MI355X_GEMM_ACT") || atoi(getenv("MI355X_GEMM_ACT")) != 0);   // read per compile
    if (!on || x->type.dt != DType::BF16 || x->users.empty() || !x->def) return false;
    Region* r = x->def->parent;
    std::unordered_set<Op*> in;
    std::vector<Op*> order;
    std::vector<Value*> work{x};
    while (!work.empty()) {
      Value* v = work.back();
      work.pop_back();
      for (Op* u : v->users) {
        if (in.count(u)) continue;
        static const std::set<std::string> el = {"add", "subtract", "multiply", "divide", "power", "tanh", "negate", "exponential", "logistic", "convert"};
        if (u->parent != r || !el.count(u->name) || u->results.size() != 1 || u->result()->type.dims != x->type.dims) {
          if (v == x) return false;     // the product itself is read from outside the chain: it has to exist in memory
          continue;                     // a reader outside the chain: v is a candidate for the chain's result
        }
        if (in.size() >= 32) return false;
        in.insert(u);
        order.push_back(u);
        work.push_back(u->result());
      }
    }
    if (in.empty()) return false;
    // exactly one value of the chain is read from outside, and it has no reader inside
    Value* out = nullptr;
    for (Op* o : order) {
      bool outside = false, inside = false;
      for (Op* u : o->result()->users) (in.count(u) ? inside : outside) = true;
      if (o->result()->users.empty()) outside = true;
      if (outside && inside) return false;
      if (outside) {
        if (out) return false;
        out = o->result();
      }
    }
    if (!out || out->type.dt != DType::BF16) return false;
    // every other input of the chain is a constant (checked by the evaluation); fit the three constants
    auto f = [&](double at, double& y) {
      std::unordered_map<Value*, double> memo;
      return evalChain(out, x, at, memo, y);
    };
    double yBig, y1, y2;
    if (!f(12.0, yBig) || !f(0.5, y1) || !f(1.0, y2)) return false;
    const double a = yBig / (2.0 * 12.0);
    if (!(a > 0.05 && a < 20.0)) return false;
    const double r1 = y1 / (a * 0.5) - 1.0, r2 = y2 / (a * 1.0) - 1.0;
    if (!(std::fabs(r1) < 1.0 && std::fabs(r2) < 1.0)) return false;
    const double u1 = std::atanh(r1), u2 = std::atanh(r2);      // c (x + b x^3) at 0.5 and 1
    // u1 = c (0.5 + 0.125 b), u2 = c (1 + b)  =>  b = (0.5 u2 - u1) / (u1 - 0.125 u2), c = u2 / (1 + b)
    const double den = u1 - 0.125 * u2;
    if (std::fabs(den) < 1e-9) return false;
    const double b = (0.5 * u2 - u1) / den;
    const double c = u2 / (1.0 + b);
    if (!(c > 0.0) || !std::isfinite(b) || !std::isfinite(c)) return false;
    for (double at : {-6.0, -3.0, -1.5, -0.7, -0.1, 0.0, 0.2, 0.9, 1.7, 2.5, 4.0, 7.0}) {
      double y;
      if (!f(at, y)) return false;
      const double want = a * at * (1.0 + std::tanh(c * (at + b * at * at * at)));
      if (!(std::fabs(y - want) <= 1e-6 * (1.0 + std::fabs(want)))) return false;
    }
    m.out = out;
    m.ops = order;
    m.a = (float)a; m.b = (float)b; m.c = (float)c;
    return true;
  }

  // ---------------------------------------------------------------- fused attention
  // dot_general(q, k) -> [* scale] -> [select(mask, ., c)] -> softmax over the keys -> convert -> dot_general(., v)
  // [-> transpose that merges the heads], every intermediate read by this chain only: one launch of the fused
  // kernel.  Matching starts from the second product and walks up.
  struct AttnMatch {
    Op* qk = nullptr;
    Op* pv = nullptr;
    Op* merge = nullptr;          // transpose [0, 2, 1, 3] of the result, if it is the only reader
    Value* mask = nullptr;        // i1, rank 4, dims 1 or full
    float scale = 1.f, masked = 0.f;
    std::vector<Op*> absorbed;    // ops between the two products (and the products)
  };

  static bool splatFloat(Value* v, float& out) {
    Op* d = v->def;
    while (d && (d->name == "broadcast_in_dim" || d->name == "reshape") && d->operands[0]->type.numel() == 1) d = d->operands[0]->def;
    if (!d || d->name != "constant") return false;
    auto& dd = *d->attrs.at("value").dense;
    if (dd.type.dt != DType::F32 || (!dd.splat && dd.type.numel() != 1)) return false;
    memcpy(&out, dd.bytes.data(), 4);
    return true;
  }

  // v = broadcast_in_dim(r, dims = [0, 1, 2]) of a reduce over dim 3 of `x` with the given reducer
  static Op* rowReduceOf(Value* v, Value* x, const char* kind, std::vector<Op*>& absorbed) {
    Op* bc = v->def;
    if (!bc || bc->name != "broadcast_in_dim" || v->users.size() != 1 || bc->ints("dims") != std::vector<int64_t>{0, 1, 2}) return nullptr;
    Op* red = bc->operands[0]->def;
    if (!red || red->name != "reduce" || bc->operands[0]->users.size() != 1 || red->operands[0] != x) return nullptr;
    const char* k = simpleReduceKind(*red);
    if (!k || std::string(k) != kind || red->ints("dimensions") != std::vector<int64_t>{3}) return nullptr;
    float init = 0.f;
    if (!splatFloat(red->operands[1], init)) return nullptr;
    if (std::string(kind) == "add" ? init != 0.f : !(init == -__builtin_inff())) return nullptr;
    absorbed.push_back(bc);
    absorbed.push_back(red);
    return red;
  }

  static bool matchAttention(Op* pv, AttnMatch& m) {
    const bool on = !strictBf16() && (!getenv("MI355X_ATTENTION") || atoi(getenv("MI355X_ATTENTION")) != 0);   // read per compile
    if (!on || pv->name != "dot_general") return false;
    Value* p = pv->operands[0];
    Value* v = pv->operands[1];
    if (p->type.dt != DType::BF16 || v->type.dt != DType::BF16 || pv->result()->type.dt != DType::BF16) return false;
    if (p->type.rank() != 4 || v->type.rank() != 4) return false;
    if (pv->ints("lhs_batch") != std::vector<int64_t>{0, 1} || pv->ints("lhs_contract") != std::vector<int64_t>{3}) return false;
    if (pv->ints("rhs_batch").size() != 2 || pv->ints("rhs_contract").size() != 1) return false;
    // the free dim of v must be its last one (the head dim, contiguous)
    {
      std::vector<bool> used(4, false);
      for (auto d : pv->ints("rhs_batch")) used[(size_t)d] = true;
      used[(size_t)pv->ints("rhs_contract")[0]] = true;
      if (used[3]) return false;
    }
    m.pv = pv;
    Op* cv = p->def;
    if (!cv || cv->name != "convert" || p->users.size() != 1 || cv->operands[0]->type.dt != DType::F32) return false;
    Value* probs = cv->operands[0];
    Op* dv = probs->def;
    if (!dv || dv->name != "divide" || probs->users.size() != 1) return false;
    Value* e = dv->operands[0];
    Op* ex = e->def;
    if (!ex || ex->name != "exponential" || e->users.size() != 2) return false;
    m.absorbed = {pv, cv, dv, ex};
    if (!rowReduceOf(dv->operands[1], e, "add", m.absorbed)) return false;
    Value* centred = ex->operands[0];
    Op* sb = centred->def;
    if (!sb || sb->name != "subtract" || centred->users.size() != 1) return false;
    m.absorbed.push_back(sb);
    Value* x = sb->operands[0];
    if (x->users.size() != 2 || !rowReduceOf(sb->operands[1], x, "maximum", m.absorbed)) return false;
    if (x->def && x->def->name == "select" && x->type.dt == DType::F32) {
      Op* sel = x->def;
      Op* mb = sel->operands[0]->def;
      float neg = 0.f;
      if (!mb || mb->name != "broadcast_in_dim" || sel->operands[0]->users.size() != 1 || mb->ints("dims") != std::vector<int64_t>{0, 1, 2, 3}) return false;
      if (!splatFloat(sel->operands[2], neg)) return false;
      Value* ms = mb->operands[0];
      if (ms->type.dt != DType::Pred || ms->type.rank() != 4) return false;
      for (int d = 0; d < 4; ++d) if (ms->type.dims[(size_t)d] != 1 && ms->type.dims[(size_t)d] != x->type.dims[(size_t)d]) return false;
      m.mask = ms;
      m.masked = neg;
      m.absorbed.push_back(sel);
      m.absorbed.push_back(mb);
      x = sel->operands[1];
      if (x->users.size() != 1) return false;
    }
    if (x->def && x->def->name == "multiply") {
      Op* mu = x->def;
      float sc = 1.f;
      Value* other = nullptr;
      if (splatFloat(mu->operands[1], sc)) other = mu->operands[0];
      else if (splatFloat(mu->operands[0], sc)) other = mu->operands[1];
      else return false;
      m.scale = sc;
      m.absorbed.push_back(mu);
      x = other;
      if (x->users.size() != 1) return false;
    }
    Op* qk = x->def;
    if (!qk || qk->name != "dot_general" || x->type.dt != DType::F32 || qk->parent != pv->parent) return false;
    Value* q = qk->operands[0];
    Value* k = qk->operands[1];
    if (q->type.dt != DType::BF16 || k->type.dt != DType::BF16 || q->type.rank() != 4 || k->type.rank() != 4) return false;
    if (qk->ints("lhs_batch").size() != 2 || qk->ints("rhs_batch").size() != 2) return false;
    if (qk->ints("lhs_contract") != std::vector<int64_t>{3} || qk->ints("rhs_contract") != std::vector<int64_t>{3}) return false;
    m.qk = qk;
    m.absorbed.push_back(qk);
    for (Op* o : m.absorbed) if (o->parent != pv->parent) return false;
    // result read only by the head-merging transpose: write it in that layout
    Value* out = pv->result();
    if (out->users.size() == 1 && out->users[0]->name == "transpose" && out->users[0]->parent == pv->parent &&
        out->users[0]->ints("dims") == std::vector<int64_t>{0, 2, 1, 3})
      m.merge = out->users[0];
    return true;
  }

  // dims of a rank-4 operand of a batched product: its two batch dims in result order, then the remaining non-contracted dim
  static void attnDims(Op* dot, bool lhs, int& db, int& dn, int& dfree) {
    auto& batch = dot->ints(lhs ? "lhs_batch" : "rhs_batch");
    int64_t contract = dot->ints(lhs ? "lhs_contract" : "rhs_contract")[0];
    db = (int)batch[0];
    dn = (int)batch[1];
    dfree = -1;
    for (int d = 0; d < 4; ++d) if (d != db && d != dn && d != contract) dfree = d;
  }

  bool emitAttention(const AttnMatch& m, Plan& plan) {
    Value* q = m.qk->operands[0];
    Value* k = m.qk->operands[1];
    Value* v = m.pv->operands[1];
    Value* out = m.merge ? m.merge->result() : m.pv->result();
    auto stored = [this](Value* x) { return hasStorage(x); };
    View vq, vk, vv;
    Value* ops3[3] = {q, k, v};
    View* views[3] = {&vq, &vk, &vv};
    Op* users[3] = {m.qk, m.qk, m.pv};
    for (int i = 0; i < 3; ++i) {
      Value* x = ops3[i];
      if (!hasStorage(x) && !(dotTakesView(x, users[i]) && resolveView(x, stored, *views[i]) && views[i]->iterOffsets.empty())) materializeNow(x, plan);
      if (hasStorage(x)) { views[i]->root = x; views[i]->offset = 0; views[i]->strides = stridesOf(x->type); }
    }
    AttentionDesc a;
    int db, dn, df;
    attnDims(m.qk, true, db, dn, df);          // q: [b, n] batch, free dim = queries, dim 3 = head
    if (df < 0 || df == 3 || vq.strides[3] != 1) return false;
    a.B = q->type.dims[(size_t)db]; a.N = q->type.dims[(size_t)dn]; a.T = q->type.dims[(size_t)df]; a.H = q->type.dims[3];
    a.qB = vq.strides[(size_t)db]; a.qN = vq.strides[(size_t)dn]; a.qT = vq.strides[(size_t)df];
    attnDims(m.qk, false, db, dn, df);
    if (df < 0 || df == 3 || vk.strides[3] != 1) return false;
    a.S = k->type.dims[(size_t)df];
    a.kB = vk.strides[(size_t)db]; a.kN = vk.strides[(size_t)dn]; a.kS = vk.strides[(size_t)df];
    {
      auto& batch = m.pv->ints("rhs_batch");
      int64_t contract = m.pv->ints("rhs_contract")[0];
      if (vv.strides[3] != 1 || v->type.dims[3] != a.H || v->type.dims[(size_t)contract] != a.S) return false;
      a.vB = vv.strides[(size_t)batch[0]]; a.vN = vv.strides[(size_t)batch[1]]; a.vS = vv.strides[(size_t)contract];
    }
    // result [b, n, t, h] dense, or [b, t, n, h] after the head merge
    if (m.merge) { a.oB = a.T * a.N * a.H; a.oT = a.N * a.H; a.oN = a.H; }
    else { a.oB = a.N * a.T * a.H; a.oN = a.T * a.H; a.oT = a.H; }
    a.scale = m.scale;
    a.masked = m.masked;
    a.hasMask = m.mask != nullptr;
    if (m.mask) {
      if (!hasStorage(m.mask)) materializeNow(m.mask, plan);
      auto ms = stridesOf(m.mask->type);
      auto md = m.mask->type.dims;
      a.mB = md[0] == 1 ? 0 : ms[0]; a.mN = md[1] == 1 ? 0 : ms[1]; a.mT = md[2] == 1 ? 0 : ms[2]; a.mS = md[3] == 1 ? 0 : ms[3];
    }
    mi355_attention_desc abi = toAbi(a);
    if (!mi355_attention_supported(&abi)) return false;
    if ((vq.offset | vk.offset | vv.offset) % 8 != 0) return false;
    int sid = newStorage(out->type.bytes());
    bind(out, sid);
    int t = ++time_;
    Step s;
    s.kind = Step::Attention;
    s.time = t;
    s.label = "attention " + q->type.str() + (m.mask ? " masked" : "") + (m.merge ? " + head merge" : "");
    s.attn = a;
    s.args = {ref(storageOf(vq.root), t), ref(storageOf(vk.root), t), ref(storageOf(vv.root), t), ref(sid, t)};
    s.args[0].offset = vq.offset * 2;
    s.args[1].offset = vk.offset * 2;
    s.args[2].offset = vv.offset * 2;
    if (m.mask) s.args.push_back(ref(storageOf(m.mask), t));
    plan.steps.push_back(std::move(s));
    for (Op* o : m.absorbed) emitted_.insert(o);
    if (m.merge) emitted_.insert(m.merge);
    return true;
  }

  void emitSort(Op* op, Plan& plan) {
    for (auto* v : op->operands) if (!hasStorage(v)) materializeNow(v, plan);
    std::vector<Value*> outs;
    for (auto& r : op->results) outs.push_back(r.get());
    if (outs.empty() || outs[0]->type.numel() == 0) {
      for (auto* o : outs) bind(o, newStorage(4));
      return;
    }
    FusedCode fc = generateSortKernel(op, leafPred());
    for (auto* o : outs) bind(o, newStorage(o->type.bytes()));
    emitted_.insert(op);
    addFused(plan, fc, "sort " + op->operands[0]->type.str() + " dim " + std::to_string(op->integer("dimension")), outs);
  }

  struct DotPlan {
    GemmDesc g;
    View va, vb;
    size_t rhsFreeDims = 0;
  };

  // materialises or resolves the operands of a dot_general and collapses its dims to one strided batched GEMM
  DotPlan prepareDot(Op* op, Plan& plan) {
    Value* a = op->operands[0];
    Value* b = op->operands[1];
    Value* c = op->result();
    std::vector<int64_t> ab = op->ints("lhs_batch"), bb = op->ints("rhs_batch"), ac = op->ints("lhs_contract"), bc = op->ints("rhs_contract");
    if (op->name == "dot") { ac = {a->type.rank() - 1}; bc = {0}; }
    auto has = [](const std::vector<int64_t>& v, int64_t x) { return std::find(v.begin(), v.end(), x) != v.end(); };
    std::vector<int64_t> af, bf;
    for (int d = 0; d < a->type.rank(); ++d) if (!has(ab, d) && !has(ac, d)) af.push_back(d);
    for (int d = 0; d < b->type.rank(); ++d) if (!has(bb, d) && !has(bc, d)) bf.push_back(d);
    if (!isFloat(a->type.dt) || a->type.dt == DType::F64 || a->type.dt == DType::F16)
      throw CompileError("dot_general: only f32 and bf16 operands are supported");
    View va, vb;
    auto stored = [this](Value* v) { return hasStorage(v); };
    DotPlan dp;
    GemmDesc& g = dp.g;
    g.inType = a->type.dt;
    g.outType = c->type.dt;
    std::vector<int64_t> bsz;
    std::vector<int64_t> abst, bbst;
    // An operand that is a chain of views over a buffer is read in place when its dims then still collapse to one
    // strided 2-D matrix per batch; otherwise the chain is written out first and read as the plain tensor it makes
    // (canonicalizeDotLayouts has put a transpose in front of every product whose plain operands would not collapse).
    for (int attempt = 0; attempt < 2; ++attempt) {
      const bool viewsAllowed = attempt == 0;
      bool usedView = false;
      for (Value* v : {a, b}) {
        View& vw = v == a ? va : vb;
        if (!hasStorage(v)) {
          if (viewsAllowed && dotTakesView(v, op) && resolveView(v, stored, vw)) usedView = true;
          else materializeNow(v, plan);
        }
        if (hasStorage(v)) { vw.root = v; vw.offset = 0; vw.strides = stridesOf(v->type); vw.iterOffsets.clear(); }
      }
      if (b == a) vb = va;
      // contraction dims: order both sides by the lhs stride so each side collapses when it can
      std::vector<size_t> order(ac.size());
      for (size_t k = 0; k < order.size(); ++k) order[k] = k;
      const std::vector<int64_t>& ast = va.strides;
      std::sort(order.begin(), order.end(), [&](size_t x, size_t y) { return ast[ac[x]] > ast[ac[y]]; });
      std::vector<int64_t> acs, bcs;
      for (auto k : order) { acs.push_back(ac[k]); bcs.push_back(bc[k]); }
      int64_t Ka = 0, Kb = 0, M = 0, N = 0;
      bool ok = mergeDims(a->type, va.strides, acs, Ka, g.aCol) && mergeDims(b->type, vb.strides, bcs, Kb, g.bRow) &&
                mergeDims(a->type, va.strides, af, M, g.aRow) && mergeDims(b->type, vb.strides, bf, N, g.bCol);
      g.M = M; g.N = N; g.K = Ka;
      // batch dims: up to two independent strides per operand
      bsz.clear(); abst.clear(); bbst.clear();
      const std::vector<int64_t>& bstr = vb.strides;
      for (size_t k = 0; k < ab.size(); ++k) {
        if (a->type.dims[ab[k]] == 1) continue;
        if (!bsz.empty() && ast[ab[k]] * a->type.dims[ab[k]] == abst.back() && bstr[bb[k]] * b->type.dims[bb[k]] == bbst.back()) {
          bsz.back() *= a->type.dims[ab[k]];
          abst.back() = ast[ab[k]];
          bbst.back() = bstr[bb[k]];
        } else {
          bsz.push_back(a->type.dims[ab[k]]);
          abst.push_back(ast[ab[k]]);
          bbst.push_back(bstr[bb[k]]);
        }
      }
      if (ok && bsz.size() <= 2 && Ka == Kb) break;
      if (!usedView)
        throw CompileError("dot_general: operand layout needs a transposed copy (dims do not collapse to strided 2-D); not supported yet: " + a->type.str() + " x " + b->type.str());
    }
    if (bsz.size() >= 1) { g.batch0 = bsz[0]; g.aB0 = abst[0]; g.bB0 = bbst[0]; }
    if (bsz.size() == 2) { g.batch1 = bsz[1]; g.aB1 = abst[1]; g.bB1 = bbst[1]; }
    dp.va = va;
    dp.vb = vb;
    dp.rhsFreeDims = bf.size();
    return dp;
  }

  // value-level form of the bias pattern: the add that follows `c` and only adds a broadcast 1-D bias over c's last dim
  static Op* biasAddOf(Value* c) {
    static const bool fuseBias = !getenv("MI355X_GEMM_BIAS") || atoi(getenv("MI355X_GEMM_BIAS")) != 0;
    if (!fuseBias || !c->def || c->users.size() != 1 || c->users[0]->name != "add" || c->users[0]->parent != c->def->parent) return nullptr;
    if (c->type.numel() == 0 || c->type.rank() == 0) return nullptr;
    Op* add = c->users[0];
    Value* other = add->operands[0] == c ? add->operands[1] : add->operands[0];
    Op* bc = other->def;
    if (other == c || !bc || bc->name != "broadcast_in_dim" || bc->parent != c->def->parent) return nullptr;
    Value* bias = bc->operands[0];
    if (bias->type.rank() != 1 || bias->type.dt != c->type.dt || bias->type.dims[0] != c->type.dims.back()) return nullptr;
    if (bc->ints("dims") != std::vector<int64_t>{(int64_t)c->type.rank() - 1}) return nullptr;
    return add;
  }

  // add(dot_general, dot_general) of two single-use f32 products with one result type: the other product, or null
  static Op* sumPartner(Op* dot) {
    static const bool on = !getenv("MI355X_GEMM_SUM") || atoi(getenv("MI355X_GEMM_SUM")) != 0;
    if (!on || dot->name != "dot_general") return nullptr;
    Value* c = dot->result();
    if (c->type.dt != DType::F32 || c->users.size() != 1 || c->users[0]->name != "add" || c->users[0]->parent != dot->parent) return nullptr;
    Op* add = c->users[0];
    Value* o = add->operands[0] == c ? add->operands[1] : add->operands[0];
    if (o == c || !o->def || o->def->name != "dot_general" || o->def->parent != dot->parent || o->users.size() != 1) return nullptr;
    if (!(o->type == c->type) || o->def->operands[0]->type.dt != DType::F32 || dot->operands[0]->type.dt != DType::F32) return nullptr;
    return o->def;
  }

  // `first` (may be null) is an earlier product that was held back because add(first, op) can be one launch
  void emitDot(Op* op, Plan& plan, Op* first = nullptr) {
    if (first) {
      DotPlan d1 = prepareDot(first, plan), d2 = prepareDot(op, plan);
      mi355_gemm_desc a1 = toAbi(d1.g), a2 = toAbi(d2.g);
      bool both = mi355_gemm_is_small(&a1) && mi355_gemm_is_small(&a2) && d1.g.M == d2.g.M && d1.g.N == d2.g.N &&
                  d1.g.batch0 == d2.g.batch0 && d1.g.batch1 == d2.g.batch1;
      if (!both) {
        emitDotStep(first, plan, d1, nullptr, nullptr);
        emitDotStep(op, plan, d2, nullptr, nullptr);
        return;
      }
      emitDotStep(first, plan, d1, op, &d2);
      return;
    }
    DotPlan d = prepareDot(op, plan);
    emitDotStep(op, plan, d, nullptr, nullptr);
  }

  void emitDotStep(Op* op, Plan& plan, const DotPlan& dp, Op* second, const DotPlan* dp2) {
    Value* a = op->operands[0];
    Value* b = op->operands[1];
    Value* c = op->result();
    const GemmDesc& g = dp.g;
    const View& va = dp.va;
    const View& vb = dp.vb;
    // the value the step produces: the product, or the sum of the two products
    Value* produced = c;
    Op* sumAdd = nullptr;
    if (second) {
      sumAdd = c->users[0];
      produced = sumAdd->result();
    }
    // product -> add(broadcast(bias over the last dim)) with no other reader of the product: the kernels add the
    // bias while they store the result (the reference fuses the same pair into one addmm, passes/fuse_bias_add.cc:120-171)
    Value* biasV = nullptr;
    Op* biasAdd = dp.rhsFreeDims == 1 ? biasAddOf(produced) : nullptr;
    if (biasAdd) {
      Value* other = biasAdd->operands[0] == produced ? biasAdd->operands[1] : biasAdd->operands[0];
      biasV = other->def->operands[0];
      if (!hasStorage(biasV)) {
        // a computed bias is materialised here only when everything it reads is already in memory
        std::unordered_set<Value*> seen;
        int leaves = 0;
        if (biasV->def && isFusibleOp(*biasV->def) && biasV->def->results.size() == 1 && leavesReady(biasV, {}, seen, leaves)) materializeNow(biasV, plan);
        else biasAdd = nullptr, biasV = nullptr;
      }
    }
    // ... -> tanh-form GELU read by nothing else: applied while the result is stored (bf16 products)
    ActMatch act;
    const bool fuseAct = !second && c->type.numel() > 0 && g.inType == DType::BF16 && g.outType == DType::BF16 &&
                         matchActivation(biasAdd ? biasAdd->result() : produced, act);
    // ... -> maximum(x, 0) read by nothing else: a small fp32 product applies it while it stores
    Op* relu = nullptr;
    {
      static const bool reluOn = !getenv("MI355X_GEMM_RELU") || atoi(getenv("MI355X_GEMM_RELU")) != 0;
      Value* x = biasAdd ? biasAdd->result() : produced;
      mi355_gemm_desc small = toAbi(g);
      if (reluOn && !fuseAct && c->type.numel() > 0 && g.inType == DType::F32 && g.outType == DType::F32 && mi355_gemm_is_small(&small) &&
          x->users.size() == 1 && x->users[0]->parent == x->def->parent) {
        Op* u = x->users[0];
        if (u->name == "maximum" && u->operands.size() == 2 && u->operands[0] != u->operands[1]) {
          float zero = 1.f;
          Value* other = u->operands[0] == x ? u->operands[1] : u->operands[0];
          if (splatFloat(other, zero) && zero == 0.f) relu = u;
        }
      }
    }
    // ... -> add(x, y) with y a tensor in memory and no other reader of the product (a gradient summed into an accumulator
    // that a loop carries): a small fp32 product adds y while it stores, in the order product + y like the add itself
    Op* accumulate = nullptr;
    Value* addendV = nullptr;
    {
      static const bool on = !getenv("MI355X_GEMM_ADDEND") || atoi(getenv("MI355X_GEMM_ADDEND")) != 0;
      mi355_gemm_desc small = toAbi(g);
      if (on && !biasAdd && !fuseAct && !relu && c->type.numel() > 0 && g.inType == DType::F32 && g.outType == DType::F32 &&
          mi355_gemm_is_small(&small) && produced->users.size() == 1 && produced->users[0]->name == "add" &&
          produced->users[0]->parent == op->parent) {
        Op* u = produced->users[0];
        Value* y = u->operands[0] == produced ? u->operands[1] : u->operands[0];
        if (y != produced && y->type == produced->type && hasStorage(y)) accumulate = u, addendV = y;
      }
    }
    int sid = newStorage(c->type.bytes());
    bind(produced, sid);
    if (sumAdd) emitted_.insert(sumAdd);
    if (c->type.numel() == 0) return;
    int t = ++time_;
    Step s;
    s.kind = Step::Gemm;
    s.time = t;
    s.label = "dot_general " + a->type.str() + " x " + b->type.str() + (second ? " + " + second->operands[0]->type.str() + " x " + second->operands[1]->type.str() : "") +
              (biasV ? " + bias" : "") + (fuseAct ? " + gelu" : "") + (relu ? " + relu" : "") + (accumulate ? " + tensor" : "");
    if (accumulate) {
      s.addend = ref(storageOf(addendV), t);
      storage_[accumulate->result()] = sid;   // the step writes the sum; nothing reads the bare product, so the buffer still holds one value
      emitted_.insert(accumulate);
    }
    s.gemm = g;
    if (relu) {
      s.gemm.act = 2;
      bind(relu->result(), sid);   // the step writes the activation; nothing reads the value before it
      emitted_.insert(relu);
    }
    if (fuseAct) {
      s.gemm.act = 1;
      s.gemm.actA = act.a; s.gemm.actB = act.b; s.gemm.actC = act.c;
      bind(act.out, sid);   // the step writes the activation; the chain's other values are never needed
      for (Op* o : act.ops) emitted_.insert(o);
    }
    s.args = {ref(storageOf(va.root), t), ref(storageOf(vb.root), t), ref(sid, t)};
    s.args[0].offset = va.offset * (int64_t)dtypeSize(a->type.dt);
    s.args[1].offset = vb.offset * (int64_t)dtypeSize(b->type.dt);
    followCounter(s.args[0], va.iterOffsets, (int64_t)dtypeSize(a->type.dt));
    followCounter(s.args[1], vb.iterOffsets, (int64_t)dtypeSize(b->type.dt));
    if (biasV) {
      s.bias = ref(storageOf(biasV), t);
      bind(biasAdd->result(), sid);   // the step writes the sum; nothing reads the bare product
      emitted_.insert(biasAdd);
    }
    if (second) {
      s.gemm2 = dp2->g;
      s.dual = true;
      s.args.push_back(ref(storageOf(dp2->va.root), t));
      s.args.push_back(ref(storageOf(dp2->vb.root), t));
      s.args[3].offset = dp2->va.offset * 4;
      s.args[4].offset = dp2->vb.offset * 4;
      followCounter(s.args[3], dp2->va.iterOffsets, 4);
      followCounter(s.args[4], dp2->vb.iterOffsets, 4);
      plan.steps.push_back(std::move(s));
      return;
    }
    // room for a k-contiguous copy of an operand that is laid out along m or n
    mi355_gemm_desc abi = toAbi(g);
    int64_t ws = ((int64_t)mi355_gemm_workspace_bytes(&abi) + kAlign - 1) / kAlign * kAlign;
    s.workspaceBytes = ws;
    if (ws > 0) s.args.push_back(ref(newStorage((size_t)ws), t));
    plan.steps.push_back(std::move(s));
  }

  void emitConv(Op* op, Plan& plan) {
    Value* lhs = op->operands[0];
    Value* rhs = op->operands[1];
    Value* out = op->result();
    std::vector<int64_t> flipped;
    if (!hasStorage(rhs) && isWindowReverse(rhs, op)) {
      flipped = rhs->def->ints("dims");
      rhs = rhs->def->operands[0];
    }
    for (Value* v : {lhs, rhs}) if (!hasStorage(v)) materializeNow(v, plan);
    const ConvDims& cd = op->convDims;
    int nsp = (int)cd.lhsSpatial.size();
    if (nsp > 3) throw CompileError("convolution with more than 3 spatial dims is not supported");
    if (lhs->type.dt != DType::F32 && lhs->type.dt != DType::BF16) throw CompileError("convolution: only f32 and bf16 are supported");
    ConvDesc c;
    c.nsp = nsp;
    c.type = lhs->type.dt;
    c.featureGroups = op->integer("feature_group_count", 1);
    c.batchGroups = op->integer("batch_group_count", 1);
    auto ls = stridesOf(lhs->type), rs = stridesOf(rhs->type), os = stridesOf(out->type);
    c.N = lhs->type.dims[cd.lhsBatch] / c.batchGroups;
    c.C = lhs->type.dims[cd.lhsFeature];
    c.O = rhs->type.dims[cd.rhsOut];
    c.lhsB = ls[cd.lhsBatch]; c.lhsF = ls[cd.lhsFeature];
    c.rhsI = rs[cd.rhsIn]; c.rhsO = rs[cd.rhsOut];
    c.outB = os[cd.outBatch]; c.outF = os[cd.outFeature];
    auto& stride = op->ints("stride");
    auto& pad = op->ints("pad");
    auto& ld = op->ints("lhs_dilate");
    auto& rd = op->ints("rhs_dilate");
    auto& rev = op->ints("reverse");
    for (int d = 0; d < nsp; ++d) {
      c.in[d] = lhs->type.dims[cd.lhsSpatial[d]];
      c.k[d] = rhs->type.dims[cd.rhsSpatial[d]];
      c.out[d] = out->type.dims[cd.outSpatial[d]];
      c.lhsS[d] = ls[cd.lhsSpatial[d]];
      c.rhsS[d] = rs[cd.rhsSpatial[d]];
      c.outS[d] = os[cd.outSpatial[d]];
      c.stride[d] = stride.empty() ? 1 : stride[d];
      c.padLo[d] = pad.empty() ? 0 : pad[2 * d];
      c.ldil[d] = ld.empty() ? 1 : ld[d];
      c.rdil[d] = rd.empty() ? 1 : rd[d];
      c.rev[d] = rev.empty() ? 0 : rev[d];
      if (std::find(flipped.begin(), flipped.end(), cd.rhsSpatial[d]) != flipped.end()) c.rev[d] = !c.rev[d];
    }
    int sid = newStorage(out->type.bytes());
    bind(out, sid);
    if (out->type.numel() == 0) return;
    int t = ++time_;
    Step s;
    s.kind = Step::Conv;
    s.label = "convolution " + lhs->type.str() + " * " + rhs->type.str();
    s.conv = c;
    s.args = {ref(storageOf(lhs), t), ref(storageOf(rhs), t), ref(sid, t)};
    s.time = t;
    // split-K partial sums for shapes with few output tiles (filter gradients, late stages)
    mi355_conv_desc abi = toAbi(c);
    int64_t ws = ((int64_t)mi355_conv_workspace_bytes(&abi) + kAlign - 1) / kAlign * kAlign;
    s.workspaceBytes = ws;
    if (ws > 0) s.args.push_back(ref(newStorage((size_t)ws), t));
    plan.steps.push_back(std::move(s));
  }

  void emitScatter(Op* op, Plan& plan) {
    if (op->operands.size() != 3) throw CompileError("variadic scatter is not supported");
    Value* operand = op->operands[0];
    Value* idx = op->operands[1];
    Value* upd = op->operands[2];
    Value* res = op->result();
    uint32_t fillBits = 0;
    bool fill = !hasStorage(operand) && scatterWritesSplat(operand, op) && splatBits(operand, fillBits);
    for (Value* v : {operand, idx, upd}) if (!hasStorage(v) && !(fill && v == operand)) materializeNow(v, plan);
    auto& uwd = op->ints("update_window_dims");
    auto& iwd = op->ints("inserted_window_dims");
    auto& sdo = op->ints("scatter_dims_to_operand_dims");
    int64_t ivd = op->integer("index_vector_dim");
    // row scatter: one index per update row, whole rows of the operand's leading dim
    bool rows = operand->type.rank() >= 1 && iwd == std::vector<int64_t>{0} && sdo == std::vector<int64_t>{0} &&
                op->ints("input_batching_dims").empty();
    int64_t nUpd = 1;
    if (rows) {
      // scatter dims of updates must be the leading dims, window dims the trailing ones covering the full row
      int nScatter = upd->type.rank() - (int)uwd.size();
      for (size_t k = 0; k < uwd.size(); ++k) if (uwd[k] != nScatter + (int64_t)k) rows = false;
      if ((int)uwd.size() != operand->type.rank() - 1) rows = false;
      for (size_t k = 0; rows && k < uwd.size(); ++k) if (upd->type.dims[uwd[k]] != operand->type.dims[1 + k]) rows = false;
      for (int d = 0; rows && d < nScatter; ++d) nUpd *= upd->type.dims[d];
      int64_t nIdx = idx->type.numel();
      if (ivd < idx->type.rank() && idx->type.dims[ivd] != 1) rows = false;
      if (nIdx != nUpd) rows = false;
    }
    const char* kind = nullptr;
    {
      auto& r = *op->regions.at(0);
      if (r.ops.size() == 1 && r.ops[0]->operands.size() == 1 && r.ops[0]->operands[0] == r.args[1].get()) kind = "set";
      else if (r.ops.size() == 2 && r.ops[0]->operands.size() == 2) {
        Op* b = r.ops[0].get();
        bool both = (b->operands[0] == r.args[0].get() && b->operands[1] == r.args[1].get()) ||
                    (b->operands[1] == r.args[0].get() && b->operands[0] == r.args[1].get());
        if (both && r.ops[1]->operands[0] == b->result()) {
          if (b->name == "add") kind = "add";
          else if (b->name == "multiply") kind = "mul";
          else if (b->name == "minimum") kind = "min";
          else if (b->name == "maximum") kind = "max";
        }
      }
    }
    if (!rows || !kind) throw CompileError("stablehlo.scatter: only whole-row scatter along dim 0 with add/set/mul/min/max bodies is supported");
    if (res->type.dt != DType::F32 && res->type.dt != DType::S32 && res->type.dt != DType::U32 && res->type.dt != DType::BF16)
      throw CompileError("stablehlo.scatter: element type not supported");
    if (idx->type.dt != DType::S32 && idx->type.dt != DType::S64 && idx->type.dt != DType::U32) throw CompileError("stablehlo.scatter: index type not supported");
    // result storage: reuse the operand's buffer when nothing else reads it
    int osid = fill ? -1 : storageOf(operand);
    int sid;
    int t = ++time_;
    bool inPlace = !fill && st_[osid].kind == BufRef::Temp && st_[osid].values == 1 && operand->users.size() == 1 && !boundToOutput_.count(osid) &&
                   !outerStorage(osid);
    if (fill) {
      sid = newStorage(res->type.bytes());
    } else if (inPlace) {
      sid = osid;
    } else {
      sid = newStorage(res->type.bytes());
      Step c;
      c.kind = Step::Copy;
      c.label = "scatter operand copy";
      c.src = ref(osid, t);
      c.dst = ref(sid, t);
      c.bytes = (int64_t)res->type.bytes();
      plan.steps.push_back(std::move(c));
      t = ++time_;
    }
    bind(res, sid);
    if (nUpd == 0) return;
    Step s;
    s.kind = Step::ScatterRows;
    s.label = std::string("scatter-") + kind + " rows" + (fill ? " into a splat" : "");
    s.scatter.fill = fill;
    s.scatter.fillBits = fillBits;
    s.scatter.numUpdates = nUpd;
    s.scatter.operandRows = operand->type.dims[0];
    s.scatter.rowElems = operand->type.numel() / std::max<int64_t>(1, operand->type.dims[0]);
    s.scatter.kind = std::string(kind) == "add" ? 0 : std::string(kind) == "set" ? 1 : std::string(kind) == "mul" ? 2 : std::string(kind) == "min" ? 3 : 4;
    s.scatter.type = res->type.dt;
    s.scatter.indexType = idx->type.dt;
    // workspace: double-buffered keys and permutation plus the radix-sort counters
    int64_t wsBytes = ((int64_t)mi355_scatter_workspace_bytes(nUpd) + kAlign - 1) / kAlign * kAlign;
    int ws = newStorage((size_t)wsBytes);
    s.workspaceBytes = wsBytes;
    s.args = {ref(sid, t), ref(storageOf(idx), t), ref(storageOf(upd), t), ref(ws, t)};
    plan.steps.push_back(std::move(s));
  }

  void emitDus(Op* op, Plan& plan) {
    Value* operand = op->operands[0];
    Value* res = op->result();
    if (!hasStorage(operand)) materializeNow(operand, plan);
    int osid = storageOf(operand);
    // in place when every other reader of the operand buffer has already been issued
    bool inPlace = st_[osid].kind == BufRef::Temp && !boundToOutput_.count(osid) && !outerStorage(osid);
    if (inPlace) {
      for (Op* u : operand->users) {
        if (u == op) continue;
        if (u->parent != op->parent) { inPlace = false; break; }
        bool before = false;
        for (auto& q : op->parent->ops) {
          if (q.get() == u) { before = true; break; }
          if (q.get() == op) break;
        }
        // a fused reader may be inlined into a kernel issued later
        bool issuesItself = !isFusibleOp(*u) || needMat_[u->result()];
        if (!before || !issuesItself) { inPlace = false; break; }
      }
      if (st_[osid].values > 1 && !operand->argOf) inPlace = false;
    }
    int sid = osid;
    if (!inPlace) {
      sid = newStorage(res->type.bytes());
      int t = ++time_;
      Step c;
      c.kind = Step::Copy;
      c.label = "dynamic_update_slice operand copy";
      c.src = ref(osid, t);
      c.dst = ref(sid, t);
      c.bytes = (int64_t)res->type.bytes();
      plan.steps.push_back(std::move(c));
    }
    bind(res, sid);
    if (op->operands[1]->type.numel() == 0) return;
    FusedCode fc = generateDusKernel(op, leafPred());
    addFused(plan, fc, "dynamic_update_slice", {op->operands[1]});
  }

  // counted loop: cond is `carry_i <cmp> const`, body returns carry_i + const, init is a constant
  // `counter` (optional) receives the carry index, start and step of the counter the trip count was read from
  using CounterInfo = LoopCounter;
  int64_t detectTripCount(Op* op, CounterInfo* counter = nullptr) { return staticTripCount(op, counter); }

  // `cond` (optional): a step whose condBuf / condMode / condType / condWant / condCount the copy takes over
  void applyCond(Step& c, const Step* cond, int t) {
    if (!cond || cond->condMode == 0) return;
    c.condBuf = ref(cond->condBuf.index, t);
    c.condMode = cond->condMode;
    c.condType = cond->condType;
    c.condWant = cond->condWant;
    c.condCount = cond->condCount;
  }
  void copyStep(Plan& plan, int src, int dst, int64_t bytes, const char* label, const Step* cond = nullptr) {
    if (src == dst) return;
    int t = ++time_;
    Step c;
    c.kind = Step::Copy;
    c.label = label;
    c.src = ref(src, t);
    c.dst = ref(dst, t);
    c.bytes = bytes;
    applyCond(c, cond, t);
    plan.steps.push_back(std::move(c));
  }

  // several copies between pairwise disjoint buffers as one launch
  void multiCopyStep(Plan& plan, const std::vector<std::array<int, 2>>& pairs, const std::vector<int64_t>& bytes, const char* label,
                     const Step* cond = nullptr) {
    std::vector<size_t> live;
    for (size_t i = 0; i < pairs.size(); ++i) if (pairs[i][0] != pairs[i][1]) live.push_back(i);
    for (size_t b = 0; b < live.size(); b += 16) {
      size_t e = std::min(live.size(), b + 16);
      if (e - b == 1) { copyStep(plan, pairs[live[b]][0], pairs[live[b]][1], bytes[live[b]], label, cond); continue; }
      int t = ++time_;
      Step c;
      c.kind = Step::Copy;
      c.label = label;
      for (size_t k = b; k < e; ++k) {
        c.args.push_back(ref(pairs[live[k]][0], t));
        c.args.push_back(ref(pairs[live[k]][1], t));
        c.copyBytes.push_back(bytes[live[k]]);
        c.bytes += bytes[live[k]];
      }
      applyCond(c, cond, t);
      plan.steps.push_back(std::move(c));
    }
  }

  // ---------------------------------------------------------------- loop carries written in place
  // A value a loop body yields normally lands in a temporary and is copied to the carry's slot at the end of the
  // iteration.  The kernel that produces it may write the slot directly when nothing still needs the old carry:
  // no step after the producer reads the slot, and the producer itself reads it (if at all) element for element
  // at the position it writes (c' = f * c + i * g).
  static bool movesData(const Op& op) {
    static const std::set<std::string> moves = {"broadcast_in_dim", "reshape", "transpose", "slice", "dynamic_slice", "pad", "concatenate", "gather",
                                                "reverse", "iota", "dynamic_update_slice", "bitcast_convert", "constant"};
    return moves.count(op.name) != 0;
  }
  static bool sameShapeElementwise(const Op& op) {
    if (!isFusibleOp(op) || op.results.size() != 1 || movesData(op)) return false;
    for (auto* o : op.operands) if (o->type.dims != op.results[0]->type.dims) return false;
    return true;
  }

  // the kernel step `w` reads `carryArg` only at the element it computes: every path from a value the step writes
  // down to the carry (through the values fused into the kernel) consists of same-shape elementwise ops
  bool writerReadsAligned(Step& w, Value* carryArg) {
    std::unordered_set<int> written;
    forEachRef(w, [&](BufRef& r, bool wr) { if (wr) written.insert(r.index); });
    std::vector<Value*> roots;
    for (auto& kv : storage_) if (written.count(kv.second) && kv.first->def) roots.push_back(kv.first);
    std::set<std::pair<Value*, bool>> seen;
    std::function<bool(Value*, bool, int)> walk = [&](Value* v, bool aligned, int depth) -> bool {
      if (v == carryArg) return aligned;
      if (depth > 0 && hasStorage(v)) return true;      // another buffer: a leaf of the kernel
      if (!seen.insert({v, aligned}).second) return true;
      Op* d = v->def;
      if (!d || !isFusibleOp(*d) || depth > 256) return d == nullptr || !isFusibleOp(*d) ? true : false;
      const bool ew = sameShapeElementwise(*d);
      for (auto* o : d->operands) if (!walk(o, aligned && ew, depth + 1)) return false;
      return true;
    };
    for (auto* r : roots) if (!walk(r, true, 0)) return false;
    return true;
  }

  static void forEachRef(Step& s, const std::function<void(BufRef&, bool)>& f) {
    for (size_t i = 0; i < s.args.size(); ++i) {
      bool writes = true;   // unknown layouts count as writes
      if (s.kind == Step::Kernel) writes = i < s.argWrites.size() ? s.argWrites[i] != 0 : true;
      else if (s.kind == Step::Gemm) writes = i == 2;
      else if (s.kind == Step::Conv) writes = i >= 2;
      else if (s.kind == Step::Attention) writes = i == 3;
      else if (s.kind == Step::Copy) writes = (i & 1) != 0;
      f(s.args[i], writes);
    }
    if (s.src.kind != BufRef::None) f(s.src, false);
    if (s.dst.kind != BufRef::None) f(s.dst, true);
    if (s.bias.kind != BufRef::None) f(s.bias, false);
    if (s.addend.kind != BufRef::None) f(s.addend, false);
    if (s.predBuf.kind != BufRef::None) f(s.predBuf, false);
    if (s.condBuf.kind != BufRef::None) f(s.condBuf, false);
    if (s.parentFlag.kind != BufRef::None) f(s.parentFlag, false);
    if (s.flagBuf.kind != BufRef::None) f(s.flagBuf, s.kind == Step::FlagInit || s.kind == Step::FlagAnd);
    for (auto& part : s.parts) forEachRef(part, f);
  }

  // true if the yielded storage `from` was redirected to the carry slot `slot` throughout `body`
  bool carryInPlace(Plan& body, int from, int slot, Value* carryArg) {
    auto dbg = [&](const char* why) { if (getenv("MI355X_VERBOSE")) fprintf(stderr, "[mi355x] carry %s (%s) stays copied: %s\n", carryArg->name.c_str(), carryArg->type.str().c_str(), why); };
    static const bool on = !getenv("MI355X_CARRY_IN_PLACE") || atoi(getenv("MI355X_CARRY_IN_PLACE")) != 0;
    if (!on || st_[from].kind != BufRef::Temp || boundToOutput_.count(from)) { dbg("not a temp"); return false; }
    int writer = -1;
    for (size_t k = 0; k < body.steps.size(); ++k) {
      Step& s = body.steps[k];
      if (s.cond || !s.bodies.empty()) { dbg("nested"); return false; }
      bool writesFrom = false;
      forEachRef(s, [&](BufRef& r, bool w) { if (r.index == from && w) writesFrom = true; });
      if (writesFrom) {
        if (writer >= 0) { dbg("two writers"); return false; }
        writer = (int)k;
      }
    }
    if (writer < 0) { dbg("no writer"); return false; }
    Step& w = body.steps[(size_t)writer];
    if (w.kind != Step::Kernel && w.kind != Step::Gemm) { dbg("writer kind"); return false; }
    bool writerReadsSlot = false, laterReadsSlot = false, partial = false;
    forEachRef(w, [&](BufRef& r, bool) { if (r.index == slot) writerReadsSlot = true; if (r.index == from && r.offset != 0) partial = true; });
    for (size_t k = (size_t)writer + 1; k < body.steps.size(); ++k)
      forEachRef(body.steps[k], [&](BufRef& r, bool) { if (r.index == slot) laterReadsSlot = true; });
    if (laterReadsSlot || partial) { dbg(laterReadsSlot ? "later step reads the slot" : "partial"); return false; }
    if (writerReadsSlot && (w.kind != Step::Kernel || !writerReadsAligned(w, carryArg))) { dbg("writer reads the slot unaligned"); return false; }
    for (auto& s : body.steps)
      forEachRef(s, [&](BufRef& r, bool) { if (r.index == from) r.index = slot; });
    st_[from].first = -1;   // no longer used: keep it out of the arena
    st_[from].last = -1;
    st_[from].uses.clear();
    return true;
  }

  void emitWhile(Op* op, Plan& plan) {
    size_t n = op->operands.size();
    for (auto* v : op->operands) if (!hasStorage(v)) materializeNow(v, plan);
    CounterInfo counter;
    int64_t trip = detectTripCount(op, &counter);
    // A top-level counted loop of modest length keeps its counter on the host (see ivArgs): only then does one graph
    // hold every iteration, which is what lets each iteration's launches carry their own addresses.
    static const bool hostCounters = !getenv("MI355X_HOST_COUNTERS") || atoi(getenv("MI355X_HOST_COUNTERS")) != 0;
    const bool hostCounter = hostCounters && trip >= 2 && trip <= kHostCounterMaxTrip && loopDepth_ == 0 && specFloors_.empty() && counter.carry >= 0 &&
                             isInt(op->operands[(size_t)counter.carry]->type.dt) && op->operands[(size_t)counter.carry]->type.numel() == 1;
    const size_t ivCarry = hostCounter ? (size_t)counter.carry : (size_t)-1;
    // With the counter on the host every iteration's launches carry their own addresses, so a carry that the body
    // overwrites as a whole can alternate between the two halves of one buffer: iteration k reads half k % 2 and
    // writes the other.  No kernel then updates a carry in place, the carries need no copies, and kernels that read
    // the old values may share a launch with the ones that write the new.  Carries updated through a window
    // (dynamic_update_slice) or passed through unchanged keep one slot.
    static const bool pingPongOn = !getenv("MI355X_CARRY_PING_PONG") || atoi(getenv("MI355X_CARRY_PING_PONG")) != 0;
    std::vector<char> pingPong(n, 0);
    std::vector<int> readHalf(n, -1), writeHalf(n, -1), finalHalf(n, -1);
    if (hostCounter && pingPongOn) {
      Region& bodyR = *op->regions[1];
      Op* bret = bodyR.terminator();
      for (size_t i = 0; i < n && bret && bret->operands.size() == n; ++i) {
        if (i == ivCarry) continue;
        Value* y = bret->operands[i];
        Op* d = y->def;
        if (!d || d->parent != &bodyR || y->type.bytes() > (size_t)64 << 20 || y->type.numel() == 0) continue;
        if (std::count(bret->operands.begin(), bret->operands.end(), y) != 1) continue;
        const bool whole = (isFusibleOp(*d) && d->name != "dynamic_update_slice" && d->name != "reshape" && !isPassThrough(*d) && d->name != "convert" &&
                            d->name != "broadcast_in_dim" && d->name != "constant") ||
                           d->name == "dot_general" || d->name == "dot" || d->name == "reduce";
        if (whole) pingPong[i] = 1;
      }
    }
    std::vector<int> slots(n);
    std::vector<std::array<int, 2>> initPairs;      // the first halves of double-buffered carries are filled by one launch
    std::vector<int64_t> initBytes;
    for (size_t i = 0; i < n; ++i) {
      Value* v = op->operands[i];
      int osid = storageOf(v);
      if (pingPong[i]) {
        const int64_t bytes = (int64_t)((v->type.bytes() + kAlign - 1) / kAlign * kAlign);
        slots[i] = newStorage((size_t)(2 * bytes));
        initPairs.push_back({osid, slots[i]});
        initBytes.push_back((int64_t)v->type.bytes());
        std::vector<int64_t> rd, wr;
        for (int64_t k = 0; k < trip; ++k) { rd.push_back((k % 2) * bytes); wr.push_back(((k + 1) % 2) * bytes); }
        P.ivTables.push_back(std::move(rd));
        readHalf[i] = newAlias(slots[i], 0, (int64_t)v->type.bytes(), (int)P.ivTables.size() - 1);
        P.ivTables.push_back(std::move(wr));
        writeHalf[i] = newAlias(slots[i], 0, (int64_t)v->type.bytes(), (int)P.ivTables.size() - 1);
        finalHalf[i] = newAlias(slots[i], (trip % 2) * bytes, (int64_t)v->type.bytes(), -1);
        continue;
      }
      bool reuse = st_[osid].kind == BufRef::Temp && st_[osid].values == 1 && v->users.size() == 1 && !boundToOutput_.count(osid) &&
                   !outerStorage(osid);
      if (reuse) slots[i] = osid;
      else {
        slots[i] = newStorage(v->type.bytes());
        copyStep(plan, osid, slots[i], (int64_t)v->type.bytes(), "loop carry init");
      }
    }
    {
      // (sources may repeat: the same zeros start several carries; then the copies stay separate)
      bool distinct = true;
      for (size_t x = 0; x < initPairs.size(); ++x) for (size_t y = x + 1; y < initPairs.size(); ++y) if (initPairs[x][0] == initPairs[y][0]) distinct = false;
      if (distinct) multiCopyStep(plan, initPairs, initBytes, "loop carry init");
      else for (size_t k = 0; k < initPairs.size(); ++k) copyStep(plan, initPairs[k][0], initPairs[k][1], initBytes[k], "loop carry init");
    }
    int tStart = ++time_;
    for (size_t i = 0; i < n; ++i) ref(slots[i], tStart);
    Step w;
    w.kind = Step::While;
    w.label = "while";
    w.tripCount = trip;
    // A loop whose trip count depends on data stays on the device: an alive flag, the condition folded into it every
    // iteration, the body run into temporaries and committed under the flag, so that the host may queue iterations
    // ahead and reads the flag once per chunk of them (the reference evaluates the condition on the host every
    // iteration: ops/control_flow.cc:504-536).
    static const bool deviceLoops = !getenv("MI355X_DEVICE_LOOPS") || atoi(getenv("MI355X_DEVICE_LOOPS")) != 0;
    const bool onDevice = trip < 0 && deviceLoops;
    int aliveSid = -1;
    if (onDevice) {
      aliveSid = newStorage(8);   // alive flag + count of iterations run
      Step f;
      f.kind = Step::FlagInit;
      f.label = "loop flag";
      f.flagBuf = ref(aliveSid, tStart);
      if (!aliveFlags_.empty()) f.parentFlag = ref(aliveFlags_.back(), tStart);
      plan.steps.push_back(std::move(f));
      aliveFlags_.push_back(aliveSid);
      specFloors_.push_back((int)st_.size());
    }
    ++loopDepth_;
    Region& cond = *op->regions[0];
    Region& body = *op->regions[1];
    for (size_t i = 0; i < n; ++i) {
      const int sid = pingPong[i] ? readHalf[i] : slots[i];
      bind(cond.args[i].get(), sid);
      bind(body.args[i].get(), sid);
    }
    const int bodyFloor = (int)st_.size();   // storages with higher ids are created by the body
    int counterEnd = -1;   // storage holding the counter's value after the last iteration
    if (hostCounter) {
      // table of the counter's values, one per iteration plus the final one
      const DType dt = op->operands[ivCarry]->type.dt;
      const size_t esz = dtypeSize(dt);
      const int64_t off = ((int64_t)P.constPool.size() + kAlign - 1) / kAlign * kAlign;
      P.constPool.resize((size_t)off + (size_t)(trip + 1) * esz);
      std::vector<int64_t> steps;
      for (int64_t k = 0; k <= trip; ++k) {
        const int64_t x = counter.init + k * counter.step;
        memcpy(P.constPool.data() + off + (size_t)k * esz, &x, esz);   // little endian: the low bytes are the value
        if (k < trip) steps.push_back(k * (int64_t)esz);
      }
      P.ivTables.push_back(std::move(steps));
      const int table = newStorage(esz, BufRef::Const);
      st_[table].offset = off;
      st_[table].ivTable = (int)P.ivTables.size() - 1;
      st_[table].ivDepth = 0;
      storage_[cond.args[ivCarry].get()] = table;
      storage_[body.args[ivCarry].get()] = table;
      counterEnd = newStorage(esz, BufRef::Const);
      st_[counterEnd].offset = off + trip * (int64_t)esz;
      IvInfo info;
      info.init = counter.init; info.step = counter.step; info.trip = trip;
      ivArgs()[body.args[ivCarry].get()] = info;
    }
    analyze(cond);
    analyze(body);
    if (hostCounter) {
      // the counter's next value is never stored: the loop does not read it back, and other readers recompute it from the table
      Value* next = body.terminator()->operands[ivCarry];
      if (next->def && next->def->parent == &body) needMat_[next] = false;
    }
    w.cond = std::make_unique<Plan>();
    emitRegion(cond, *w.cond);
    Value* pred = cond.terminator()->operands.at(0);
    if (!hasStorage(pred)) materializeNow(pred, *w.cond);
    w.predBuf = ref(storageOf(pred), ++time_);
    Step commit;   // carries are written only while the flag is set
    if (onDevice) {
      Step a;
      a.kind = Step::FlagAnd;
      a.label = "loop flag &= condition";
      int t = ++time_;
      a.flagBuf = ref(aliveSid, t);
      a.predBuf = ref(storageOf(pred), t);
      w.cond->steps.push_back(std::move(a));
      commit.condMode = 1;
      commit.condBuf.index = aliveSid;
    }
    auto bodyPlan = std::make_unique<Plan>();
    emitRegion(body, *bodyPlan);
    Op* ret = body.terminator();
    if (ret->operands.size() != n) throw CompileError("while: body returns the wrong number of values");
    std::vector<int> src(n);
    for (size_t i = 0; i < n; ++i) {
      if (i == ivCarry) { src[i] = slots[i]; continue; }   // never written inside the loop
      Value* v = ret->operands[i];
      if (!hasStorage(v)) materializeNow(v, *bodyPlan);
      src[i] = storageOf(v);
      if (!pingPong[i]) continue;
      // the producer writes the other half directly when the value has a buffer of its own made in this body;
      // otherwise one copy moves it there
      const int from = src[i];
      const bool own = from >= bodyFloor && st_[from].kind == BufRef::Temp && st_[from].aliasOf < 0 && st_[from].values == 1 &&
                       st_[from].bytes <= st_[writeHalf[i]].bytes + (int64_t)kAlign;
      if (own) {
        std::function<void(Plan&)> redirect = [&](Plan& p) {
          for (auto& st : p.steps) {
            forEachRef(st, [&](BufRef& r, bool) { if (r.index == from) { r.index = writeHalf[i]; r.ivTable = st_[writeHalf[i]].ivTable; r.ivDepth = 0; } });
            if (st.cond) redirect(*st.cond);
            for (auto& b : st.bodies) redirect(*b);
          }
        };
        redirect(*bodyPlan);
        for (int t : st_[from].uses) ref(slots[i], t);
        st_[from].uses.clear();
        st_[from].first = st_[from].last = -1;
        storage_[v] = writeHalf[i];
      } else {
        copyStep(*bodyPlan, from, writeHalf[i], (int64_t)v->type.bytes(), "loop carry to its other half");
      }
      src[i] = slots[i];
    }
    // carries whose producer can write the slot itself need no copy
    for (size_t i = 0; i < n; ++i) {
      if (src[i] == slots[i]) continue;
      if (std::count(src.begin(), src.end(), src[i]) != 1) continue;
      if (std::find(slots.begin(), slots.end(), src[i]) != slots.end()) continue;
      // another carry receives the old value of this slot (a swap): the copies at the end still need it
      bool slotIsSource = false;
      for (size_t j = 0; j < n; ++j) if (j != i && src[j] == slots[i]) slotIsSource = true;
      if (slotIsSource) continue;
      if (onDevice) continue;   // iterations past the end run too and must not touch the carries
      if (carryInPlace(*bodyPlan, src[i], slots[i], body.args[i].get())) {
        storage_[ret->operands[i]] = slots[i];
        src[i] = slots[i];
      }
    }
    // phase 1: values that live in another carry slot are staged through temporaries
    std::vector<std::array<int, 2>> stage, update;
    std::vector<int64_t> stageBytes, updateBytes;
    for (size_t i = 0; i < n; ++i) {
      if (src[i] == slots[i]) continue;
      bool isSlot = std::find(slots.begin(), slots.end(), src[i]) != slots.end();
      if (isSlot || st_[src[i]].kind != BufRef::Temp) {
        int tmp = newStorage(op->operands[i]->type.bytes());
        stage.push_back({src[i], tmp});
        stageBytes.push_back((int64_t)op->operands[i]->type.bytes());
        src[i] = tmp;
      }
    }
    multiCopyStep(*bodyPlan, stage, stageBytes, "loop carry stage");
    // phase 2: sources are temporaries now, destinations are distinct slots: one launch moves them all
    for (size_t i = 0; i < n; ++i) {
      update.push_back({src[i], slots[i]});
      updateBytes.push_back((int64_t)op->operands[i]->type.bytes());
    }
    multiCopyStep(*bodyPlan, update, updateBytes, "loop carry update", onDevice ? &commit : nullptr);
    int tEnd = ++time_;
    for (size_t i = 0; i < n; ++i) ref(slots[i], tEnd);
    --loopDepth_;
    if (hostCounter) ivArgs().erase(body.args[ivCarry].get());   // the registry outlives this compile: nothing stale may stay in it
    if (onDevice) {
      w.flagBuf = ref(aliveSid, tEnd);
      aliveFlags_.pop_back();
      specFloors_.pop_back();
    }
    loops_.push_back({tStart, tEnd});
    w.bodies.push_back(std::move(bodyPlan));
    w.hostCounter = hostCounter;
    for (size_t i = 0; i < n; ++i) bind(op->results[i].get(), i == ivCarry ? counterEnd : pingPong[i] ? finalHalf[i] : slots[i]);
    plan.steps.push_back(std::move(w));
  }

  void emitCase(Op* op, Plan& plan) {
    Value* index = op->operands[0];
    if (!hasStorage(index)) materializeNow(index, plan);
    int tStart = ++time_;
    Step c;
    c.kind = Step::Case;
    c.label = "case";
    c.predBuf = ref(storageOf(index), tStart);
    c.predType = index->type.dt;
    std::vector<int> outs;
    for (auto& r : op->results) outs.push_back(newStorage(r->type.bytes()));
    // Inside a loop a case with small branches runs all of them and keeps the selected results (copies conditional on
    // the index, decided on the device), so that the loop body needs no host round trip and stays one launch sequence.
    static const bool deviceCases = !getenv("MI355X_DEVICE_CASES") || atoi(getenv("MI355X_DEVICE_CASES")) != 0;
    int branchOps = 0;
    for (auto& rg : op->regions) branchOps += countOps(*rg);
    c.predicated = deviceCases && loopDepth_ > 0 && branchOps <= 96;
    if (c.predicated) specFloors_.push_back((int)st_.size());
    Step select;
    select.condMode = c.predicated ? 2 : 0;
    select.condBuf.index = storageOf(index);
    select.condType = index->type.dt;
    select.condCount = (int64_t)op->regions.size();
    for (size_t b = 0; b < op->regions.size(); ++b) {
      auto& rg = op->regions[b];
      analyze(*rg);
      auto bp = std::make_unique<Plan>();
      emitRegion(*rg, *bp);
      Op* ret = rg->terminator();
      select.condWant = (int64_t)b;
      std::vector<std::array<int, 2>> pairs;
      std::vector<int64_t> sizes;
      for (size_t k = 0; k < op->results.size(); ++k) {
        Value* v = ret->operands.at(k);
        if (!hasStorage(v)) materializeNow(v, *bp);
        pairs.push_back({storageOf(v), outs[k]});
        sizes.push_back((int64_t)v->type.bytes());
      }
      // results of one branch may share a source (the same value returned twice): single copies then
      bool distinct = true;
      for (size_t x = 0; x < pairs.size(); ++x) for (size_t y = x + 1; y < pairs.size(); ++y) if (pairs[x][0] == pairs[y][0]) distinct = false;
      if (distinct) multiCopyStep(*bp, pairs, sizes, "case result", c.predicated ? &select : nullptr);
      else for (size_t k = 0; k < pairs.size(); ++k) copyStep(*bp, pairs[k][0], pairs[k][1], sizes[k], "case result", c.predicated ? &select : nullptr);
      c.bodies.push_back(std::move(bp));
    }
    if (c.predicated) specFloors_.pop_back();
    int tEnd = ++time_;
    for (auto o : outs) { ref(o, tStart); ref(o, tEnd); }
    loops_.push_back({tStart, tEnd});
    for (size_t k = 0; k < op->results.size(); ++k) bind(op->results[k].get(), outs[k]);
    plan.steps.push_back(std::move(c));
  }

  // ---------------------------------------------------------------- horizontal batching
  // Consecutive kernel steps that touch disjoint buffers (or only read the shared ones) run as
  // the segments of one launch: small kernels cost a launch each whatever their size, and the
  // optimiser updates of a training step or the bookkeeping of a loop body come in such runs.
  static constexpr int64_t kHostCounterMaxTrip = 512;
  static constexpr unsigned kBatchMaxBlocks = 4096;   // bigger kernels fill the chip on their own
  static constexpr size_t kBatchMaxArgs = 192;
  static constexpr size_t kBatchMaxSegments = 24;

  static constexpr unsigned kBatchMaxBigBlocks = 1u << 20;   // one member of a group may be this big: small neighbours ride in its launch
  bool batchCandidate(const Step& s) const {
    return s.kind == Step::Kernel && s.grid[1] == 1 && s.grid[2] == 1 && s.block[0] == 256 && s.block[1] == 1 && s.block[2] == 1 &&
           s.grid[0] <= kBatchMaxBigBlocks && s.argWrites.size() == s.args.size() && batchableKernel(P.kernels[s.kernel].source);
  }

  // the shared prelude never declares LDS, so any __shared__ after the kernel header belongs to the body
  static bool ldsInBody(const std::string& source) {
    size_t header = source.find("extern \"C\" __global__");
    return header != std::string::npos && source.find("__shared__", header) != std::string::npos;
  }

  static bool independent(const Step& a, const Step& b) {
    for (size_t i = 0; i < a.args.size(); ++i)
      for (size_t j = 0; j < b.args.size(); ++j)
        if (a.args[i].index == b.args[j].index && (a.argWrites[i] || b.argWrites[j])) return false;
    return true;
  }

  static bool stepsIndependent(Step& a, Step& b) {
    std::vector<std::pair<int, bool>> ra, rb;
    forEachRef(a, [&](BufRef& r, bool w) { ra.push_back({r.index, w}); });
    forEachRef(b, [&](BufRef& r, bool w) { rb.push_back({r.index, w}); });
    for (auto& x : ra) for (auto& y : rb) if (x.first == y.first && (x.second || y.second)) return false;
    return true;
  }

  // Inside a loop body, a small kernel followed by a product it has nothing to do with moves behind the product, next
  // to the kernel that follows: the two kernels can then share a launch (the bookkeeping writes of a scan step beside
  // the kernel that computes the new state).
  void sinkKernelsInLoops(Plan& plan, bool inLoop) {
    for (auto& s : plan.steps) for (auto& b : s.bodies) sinkKernelsInLoops(*b, s.kind == Step::While);
    static const bool everywhere = !getenv("MI355X_SINK_TOP_LEVEL") || atoi(getenv("MI355X_SINK_TOP_LEVEL")) != 0;
    if (!inLoop && !(everywhere && &plan == &P.plan)) return;
    auto& steps = plan.steps;
    for (int i = (int)steps.size() - 2; i >= 0; --i) {
      if (!batchCandidate(steps[(size_t)i]) || steps[(size_t)i + 1].kind == Step::Kernel) continue;
      // the kernels just before it that can share its launch move with it, or none moves (splitting them would add a launch)
      int first = i;
      while (first > 0 && i - first + 1 < (int)kBatchMaxSegments && batchCandidate(steps[(size_t)first - 1])) {
        bool apart = true;
        for (int k = first; k <= i && apart; ++k) apart = stepsIndependent(steps[(size_t)first - 1], steps[(size_t)k]);
        if (!apart) break;
        --first;
      }
      auto runIndependentOf = [&](Step& other) {
        for (int k = first; k <= i; ++k) if (!stepsIndependent(steps[(size_t)k], other)) return false;
        return true;
      };
      size_t j = (size_t)i + 1;
      while (j < steps.size() && steps[j].kind != Step::Kernel && steps[j].kind != Step::While && steps[j].kind != Step::Case &&
             runIndependentOf(steps[j])) ++j;
      if (j == (size_t)i + 1 || j >= steps.size() || !batchCandidate(steps[j]) || !runIndependentOf(steps[j])) { i = first; continue; }
      // the moved kernels' buffers now live until their new neighbour runs
      for (int k = first; k <= i; ++k) {
        for (auto& a : steps[(size_t)k].args) ref(a.index, steps[j].time);
        steps[(size_t)k].time = steps[j].time;
      }
      std::rotate(steps.begin() + first, steps.begin() + i + 1, steps.begin() + (long)j);
      i = first;
    }
  }

  void batchKernels(Plan& plan) {
    std::vector<Step> out;
    auto& steps = plan.steps;
    size_t i = 0;
    while (i < steps.size()) {
      for (auto& b : steps[i].bodies) batchKernels(*b);
      if (!batchCandidate(steps[i])) { out.push_back(std::move(steps[i++])); continue; }
      size_t j = i + 1, nargs = steps[i].args.size();
      // static LDS of the segments adds up in the combined kernel: at most four segments that use any
      auto usesLds = [&](const Step& st) { return ldsInBody(P.kernels[st.kernel].source); };
      size_t ldsSegments = usesLds(steps[i]) ? 1 : 0;
      size_t bigSegments = steps[i].grid[0] > kBatchMaxBlocks ? 1 : 0;
      while (j < steps.size() && j - i < kBatchMaxSegments && batchCandidate(steps[j]) && nargs + steps[j].args.size() <= kBatchMaxArgs) {
        if (steps[j].grid[0] > kBatchMaxBlocks) { if (bigSegments >= 1) break; ++bigSegments; }
        if (usesLds(steps[j])) { if (ldsSegments >= 4) break; ++ldsSegments; }
        bool ok = true;
        for (size_t k = i; k < j && ok; ++k) ok = independent(steps[k], steps[j]);
        if (!ok) break;
        nargs += steps[j].args.size();
        ++j;
      }
      if (j - i < 2) { out.push_back(std::move(steps[i++])); continue; }
      std::vector<const std::string*> sources;
      std::vector<unsigned> grids;
      for (size_t k = i; k < j; ++k) { sources.push_back(&P.kernels[steps[k].kernel].source); grids.push_back(steps[k].grid[0]); }
      std::string combined = combineKernels(sources, grids);
      if (combined.empty()) { out.push_back(std::move(steps[i++])); continue; }
      Step m;
      m.kind = Step::Kernel;
      m.kernel = kernelId(combined);
      m.block[0] = 256;
      m.grid[0] = 0;
      m.time = steps[i].time;
      m.label = "batch[" + std::to_string(j - i) + "]:" + steps[i].label;
      const int tFirst = steps[i].time, tLast = steps[j - 1].time;
      for (size_t k = i; k < j; ++k) {
        m.grid[0] += steps[k].grid[0];
        m.algoBytes += steps[k].algoBytes;
        for (size_t a = 0; a < steps[k].args.size(); ++a) {
          m.args.push_back(steps[k].args[a]);
          m.argWrites.push_back(steps[k].argWrites[a]);
          // every buffer of the group is live for the whole group: the segments run concurrently
          ref(steps[k].args[a].index, tFirst);
          ref(steps[k].args[a].index, tLast);
        }
      }
      out.push_back(std::move(m));
      i = j;
    }
    steps = std::move(out);
  }

  // Consecutive small fp32 products that do not depend on each other (the weight and input gradients of a
  // recurrent step, say) share one launch.
  static int smallClass(const Step& s) {
    if (s.kind != Step::Gemm || s.workspaceBytes != 0 || s.gemm.inType != DType::F32 || s.gemm.outType != DType::F32) return 0;
    mi355_gemm_desc d = toAbi(s.gemm);
    int t = mi355_gemm_is_small(&d);
    if (t && s.dual) { mi355_gemm_desc d2 = toAbi(s.gemm2); if (mi355_gemm_is_small(&d2) == 0) return 0; }
    return t;
  }

  static bool gemmsIndependent(const Step& a, const Step& b) {
    auto reads = [](const Step& s) {
      std::vector<int> r{s.args[0].index, s.args[1].index};
      if (s.dual) { r.push_back(s.args[3].index); r.push_back(s.args[4].index); }
      if (s.bias.kind != BufRef::None) r.push_back(s.bias.index);
      if (s.addend.kind != BufRef::None) r.push_back(s.addend.index);
      return r;
    };
    const int wa = a.args[2].index, wb = b.args[2].index;
    if (wa == wb) return false;
    for (int x : reads(a)) if (x == wb) return false;
    for (int x : reads(b)) if (x == wa) return false;
    return true;
  }

  void groupSmallGemms(Plan& plan) {
    static const bool on = !getenv("MI355X_GEMM_GROUPS") || atoi(getenv("MI355X_GEMM_GROUPS")) != 0;
    if (!on) return;
    std::vector<Step> out;
    auto& steps = plan.steps;
    size_t i = 0;
    while (i < steps.size()) {
      for (auto& b : steps[i].bodies) groupSmallGemms(*b);
      const int cls = smallClass(steps[i]);
      size_t j = i + 1;
      if (cls) {
        while (j < steps.size() && j - i < 4 && smallClass(steps[j]) == cls) {
          bool ok = true;
          for (size_t k = i; k < j && ok; ++k) ok = gemmsIndependent(steps[k], steps[j]);
          if (!ok) break;
          ++j;
        }
      }
      if (j - i < 2) { out.push_back(std::move(steps[i++])); continue; }
      Step m;
      m.kind = Step::GemmGroup;
      m.time = steps[i].time;
      m.label = "small products x" + std::to_string(j - i);
      const int tFirst = steps[i].time, tLast = steps[j - 1].time;
      for (size_t k = i; k < j; ++k) {
        for (auto& a : steps[k].args) { ref(a.index, tFirst); ref(a.index, tLast); }
        if (steps[k].bias.kind != BufRef::None) { ref(steps[k].bias.index, tFirst); ref(steps[k].bias.index, tLast); }
        m.parts.push_back(std::move(steps[k]));
      }
      out.push_back(std::move(m));
      i = j;
    }
    steps = std::move(out);
  }

  // Convolutions whose results are not needed for several steps (filter gradients: only the optimizer update at the
  // end of the step reads them) are marked to run on a second stream.  Every buffer such a step touches then stays
  // allocated to the end of the plan, because the steps after it no longer wait for it before reusing memory.
  void forkDistantConvolutions(Plan& plan) {
    static const int minDistance = getenv("MI355X_FORK_DISTANCE") ? atoi(getenv("MI355X_FORK_DISTANCE")) : 6;
    if (minDistance <= 0) return;
    for (auto& s : plan.steps) if (s.kind == Step::While || s.kind == Step::Case) return;   // loops replay from graphs on one stream
    const size_t n = plan.steps.size();
    for (size_t i = 0; i < n; ++i) {
      Step& s = plan.steps[i];
      if (s.kind != Step::Conv || s.statsArg >= 0) continue;
      std::unordered_set<int> reads, writes;
      forEachRef(s, [&](BufRef& r, bool w) { (w ? writes : reads).insert(r.index); });
      size_t j = i + 1;
      for (; j < n; ++j) {
        bool touches = false;
        forEachRef(plan.steps[j], [&](BufRef& r, bool w) {
          if (writes.count(r.index) || (w && reads.count(r.index))) touches = true;
        });
        if (touches) break;
      }
      if (j - i < (size_t)minDistance) continue;
      s.forkId = plan.numForks++;
      if (j < n) plan.steps[j].joins.push_back(s.forkId);
      for (int sid : reads) if (st_[sid].kind == BufRef::Temp) st_[sid].last = std::max(st_[sid].last, time_);
      for (int sid : writes) if (st_[sid].kind == BufRef::Temp) st_[sid].last = std::max(st_[sid].last, time_);
    }
  }

  // ---------------------------------------------------------------- arena
  void assignArena() {
    // a buffer that is used inside a loop but defined outside it lives until the loop ends
    for (auto& s : st_) {
      if (s.kind != BufRef::Temp || s.first < 0) continue;
      for (int u : s.uses) {
        for (auto& lp : loops_) {
          if (u > lp.first && u < lp.second && !(s.first > lp.first && s.first < lp.second)) s.last = std::max(s.last, lp.second);
        }
      }
      for (auto& lp : loops_) if (s.last > lp.first && s.last < lp.second && !(s.first > lp.first)) s.last = std::max(s.last, lp.second);
    }
    std::vector<int> order;
    for (int i = 0; i < (int)st_.size(); ++i) if (st_[i].kind == BufRef::Temp && st_[i].first >= 0) order.push_back(i);
    std::sort(order.begin(), order.end(), [&](int a, int b) { return st_[a].first != st_[b].first ? st_[a].first < st_[b].first : st_[a].bytes > st_[b].bytes; });
    struct Live { int64_t off, size; int last; };
    std::vector<Live> live;
    int64_t peak = 0;
    for (int id : order) {
      Storage& s = st_[id];
      live.erase(std::remove_if(live.begin(), live.end(), [&](const Live& l) { return l.last < s.first; }), live.end());
      std::sort(live.begin(), live.end(), [](const Live& a, const Live& b) { return a.off < b.off; });
      int64_t size = (s.bytes + kAlign - 1) / kAlign * kAlign;
      int64_t off = 0;
      for (auto& l : live) {
        if (off + size <= l.off) break;
        off = std::max(off, l.off + l.size);
      }
      s.offset = off;
      live.push_back({off, size, s.last});
      peak = std::max(peak, off + size);
    }
    P.arenaBytes = peak;
  }

  BufRef finalRef(const BufRef& r) {
    if (r.kind == BufRef::None) return r;
    const Storage& s = st_[r.index];
    BufRef o;
    o.kind = s.kind;
    if (s.aliasOf >= 0) {
      const Storage& parent = st_[s.aliasOf];
      o.kind = parent.kind;
      o.index = (parent.kind == BufRef::Param || parent.kind == BufRef::Output) ? parent.index : 0;
      o.offset = ((parent.kind == BufRef::Param || parent.kind == BufRef::Output) ? 0 : parent.offset) + s.aliasOffset + r.offset;
    } else if (s.kind == BufRef::Param || s.kind == BufRef::Output) { o.index = s.index; o.offset = r.offset; }
    else { o.index = 0; o.offset = s.offset + r.offset; }
    o.ivTable = r.ivTable;
    o.ivDepth = r.ivDepth;
    return o;
  }

  void patch(Plan& plan) {
    for (auto& s : plan.steps) {
      for (auto& part : s.parts) {
        for (auto& a : part.args) a = finalRef(a);
        part.bias = finalRef(part.bias);
        part.addend = finalRef(part.addend);
      }
      for (auto& a : s.args) a = finalRef(a);
      s.src = finalRef(s.src);
      s.dst = finalRef(s.dst);
      s.bias = finalRef(s.bias);
      s.addend = finalRef(s.addend);
      s.predBuf = finalRef(s.predBuf);
      s.condBuf = finalRef(s.condBuf);
      s.flagBuf = finalRef(s.flagBuf);
      s.parentFlag = finalRef(s.parentFlag);
      if (s.cond) patch(*s.cond);
      for (auto& b : s.bodies) patch(*b);
    }
  }

  static int countSteps(const Plan& p) {
    int n = 0;
    for (auto& s : p.steps) {
      ++n;
      if (s.cond) n += countSteps(*s.cond);
      for (auto& b : s.bodies) n += countSteps(*b);
    }
    return n;
  }

  void dumpPlan(const Plan& p, int indent) {
    std::ostringstream o;
    static const char* kinds[] = {"kernel", "gemm", "conv", "scatter", "copy", "fill", "while", "case", "gemm-group", "attention", "flag-init", "flag-and"};
    for (auto& s : p.steps) {
      o << std::string(indent, ' ') << kinds[s.kind] << " " << s.label;
      if (s.kind == Step::Kernel) o << " k" << s.kernel << " grid " << s.grid[0] << "x" << s.grid[1] << " bytes " << s.algoBytes;
      if (s.kind == Step::While) o << " trip " << s.tripCount << (s.flagBuf.kind != BufRef::None ? " on-device" : "");
      if (s.kind == Step::Case && s.predicated) o << " all-branches";
      if (s.kind == Step::Copy && s.condMode) o << (s.condMode == 1 ? " if-alive" : " if-selected");
      if (s.forkId >= 0) o << " [second stream #" << s.forkId << "]";
      for (int id : s.joins) o << " [waits for #" << id << "]";
      if (getenv("MI355X_DUMP_PLAN") && atoi(getenv("MI355X_DUMP_PLAN")) >= 2) {   // what the step reads and writes
        static const char* where[] = {"none", "param", "out", "temp", "const"};
        forEachRef(const_cast<Step&>(s), [&](BufRef& r, bool wr) { o << (wr ? " W:" : " R:") << where[r.kind] << r.index << "+" << r.offset; });
      }
      o << "\n";
      P.dump += o.str();
      o.str("");
      if (s.cond) dumpPlan(*s.cond, indent + 2);
      for (auto& b : s.bodies) dumpPlan(*b, indent + 2);
      for (auto& part : s.parts) { P.dump += std::string(indent + 2, ' ') + part.label + "\n"; }
    }
  }
};

}  // namespace

int abiDtypeCode(DType d) {
  switch (d) {
    case DType::F32: return 0;
    case DType::BF16: return 1;
    case DType::S32: return 2;
    case DType::U32: return 3;
    default: return -1;
  }
}

mi355_gemm_desc toAbi(const GemmDesc& g) {
  mi355_gemm_desc d;
  d.batch0 = g.batch0; d.batch1 = g.batch1; d.M = g.M; d.N = g.N; d.K = g.K;
  d.aB0 = g.aB0; d.aB1 = g.aB1; d.aRow = g.aRow; d.aCol = g.aCol;
  d.bB0 = g.bB0; d.bB1 = g.bB1; d.bRow = g.bRow; d.bCol = g.bCol;
  d.in_dtype = abiDtypeCode(g.inType);
  d.out_dtype = abiDtypeCode(g.outType);
  d.act = g.act; d.act_a = g.actA; d.act_b = g.actB; d.act_c = g.actC;
  return d;
}

mi355_attention_desc toAbi(const AttentionDesc& a) {
  mi355_attention_desc d;
  d.B = a.B; d.N = a.N; d.T = a.T; d.S = a.S; d.H = a.H;
  d.qB = a.qB; d.qN = a.qN; d.qT = a.qT; d.kB = a.kB; d.kN = a.kN; d.kS = a.kS; d.vB = a.vB; d.vN = a.vN; d.vS = a.vS;
  d.oB = a.oB; d.oN = a.oN; d.oT = a.oT; d.mB = a.mB; d.mN = a.mN; d.mT = a.mT; d.mS = a.mS;
  d.scale = a.scale; d.masked = a.masked;
  return d;
}

mi355_conv_desc toAbi(const ConvDesc& c) {
  mi355_conv_desc d;
  memset(&d, 0, sizeof d);
  d.nsp = c.nsp; d.N = c.N; d.C = c.C; d.O = c.O;
  for (int k = 0; k < 3; ++k) {
    d.in[k] = c.in[k]; d.k[k] = c.k[k]; d.out[k] = c.out[k]; d.stride[k] = c.stride[k]; d.padLo[k] = c.padLo[k];
    d.ldil[k] = c.ldil[k]; d.rdil[k] = c.rdil[k]; d.rev[k] = c.rev[k];
    d.lhsS[k] = c.lhsS[k]; d.rhsS[k] = c.rhsS[k]; d.outS[k] = c.outS[k];
  }
  d.featureGroups = c.featureGroups; d.batchGroups = c.batchGroups;
  d.lhsB = c.lhsB; d.lhsF = c.lhsF; d.rhsI = c.rhsI; d.rhsO = c.rhsO; d.outB = c.outB; d.outF = c.outF;
  d.dtype = abiDtypeCode(c.type);
  return d;
}

std::unique_ptr<CompiledProgram> compileProgram(std::unique_ptr<Module> module) {
  auto prog = std::make_unique<CompiledProgram>();
  if (Func* mainFn = module->main()) {
    prog->paramDonation = mainFn->argDonation;
    prog->paramDonation.resize(mainFn->body.args.size(), -1);
  }
  lowerFusedOpCalls(*module);
  inlineCalls(*module);
  lowerSingleDeviceOps(*module);
  lowerIntegerDots(*module);
  widenHalfProducts(*module);
  widenScatterTypes(*module);
  lowerBitcastWidths(*module);
  lowerGeneralScatters(*module);
  lowerWindowOps(*module);
  lowerRng(*module);
  lowerTopK(*module);
  lowerEmptyReductions(*module);
  canonicalizeDotLayouts(*module);
  hoistLoopProducts(*module);
  dropScatterIndexMasks(*module);
  reluMasksFromActivations(*module);
  checkSupported(*module);
  eliminateDeadCode(module->main()->body);
  prog->module = std::move(module);
  Planner planner(*prog);
  planner.run();
  return prog;
}

}  // namespace mi355
