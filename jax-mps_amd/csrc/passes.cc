// Module-level passes run once at PJRT_Client_Compile: call inlining, dead-code
// elimination and the supported-op check.  The reference does the same three
// things with MLIR's inliner + SymbolDCE and its handler-table scan (reference:
// src/pjrt_plugin/stablehlo_parser.cc:129-149, 167-184).
#include <functional>
#include <cstring>
#include <set>
#include <unordered_map>
#include <unordered_set>

#include "ir.h"

namespace mi355 {

namespace {

using VMap = std::unordered_map<Value*, Value*>;

std::unique_ptr<Op> cloneOp(const Op& src, VMap& map, int& nextId);

std::unique_ptr<Region> cloneRegion(const Region& src, Op* parent, VMap& map, int& nextId) {
  auto r = std::make_unique<Region>();
  r->parent = parent;
  for (auto& a : src.args) {
    auto v = std::make_unique<Value>();
    v->id = nextId++;
    v->type = a->type;
    v->name = a->name;
    v->argOf = r.get();
    v->defIndex = a->defIndex;
    map[a.get()] = v.get();
    r->args.push_back(std::move(v));
  }
  for (auto& o : src.ops) {
    auto c = cloneOp(*o, map, nextId);
    c->parent = r.get();
    r->ops.push_back(std::move(c));
  }
  return r;
}

std::unique_ptr<Op> cloneOp(const Op& src, VMap& map, int& nextId) {
  auto op = std::make_unique<Op>();
  op->name = src.name;
  op->attrs = src.attrs;
  op->convDims = src.convDims;
  op->line = src.line;
  for (auto* v : src.operands) {
    auto it = map.find(v);
    op->operands.push_back(it == map.end() ? v : it->second);
  }
  for (auto& r : src.results) {
    auto v = std::make_unique<Value>();
    v->id = nextId++;
    v->type = r->type;
    v->name = r->name;
    v->def = op.get();
    v->defIndex = r->defIndex;
    map[r.get()] = v.get();
    op->results.push_back(std::move(v));
  }
  for (auto& r : src.regions) op->regions.push_back(cloneRegion(*r, op.get(), map, nextId));
  return op;
}

int maxValueId(const Region& r) {
  int m = -1;
  for (auto& a : r.args) m = std::max(m, a->id);
  for (auto& o : r.ops) {
    for (auto& v : o->results) m = std::max(m, v->id);
    for (auto& sub : o->regions) m = std::max(m, maxValueId(*sub));
  }
  return m;
}

void applyReplacements(Region& r, const VMap& repl) {
  auto resolve = [&](Value* v) {
    auto it = repl.find(v);
    while (it != repl.end()) {
      v = it->second;
      it = repl.find(v);
    }
    return v;
  };
  for (auto& o : r.ops) {
    for (auto& v : o->operands) v = resolve(v);
    for (auto& sub : o->regions) applyReplacements(*sub, repl);
  }
}

bool inlineRegion(Module& m, Region& r, VMap& repl, int& nextId, int depth) {
  if (depth > 64) throw CompileError("call inlining exceeded depth 64 (recursive functions are not supported)");
  bool any = false;
  for (size_t k = 0; k < r.ops.size(); ++k) {
    Op* op = r.ops[k].get();
    for (auto& sub : op->regions) any |= inlineRegion(m, *sub, repl, nextId, depth);
    // a composite runs its decomposition function (reference: ops/control_flow.cc:2242-2262)
    if (op->name != "call" && op->name != "composite") continue;
    const std::string& target = op->name == "call" ? op->str("callee") : op->str("decomposition");
    Func* callee = m.find(target);
    if (!callee) throw CompileError(op->name + " of unknown function @" + target);
    if (callee->body.args.size() != op->operands.size()) throw CompileError("call @" + callee->name + ": argument count mismatch");
    VMap map;
    for (size_t a = 0; a < op->operands.size(); ++a) map[callee->body.args[a].get()] = op->operands[a];
    std::vector<std::unique_ptr<Op>> cloned;
    for (auto& o : callee->body.ops) cloned.push_back(cloneOp(*o, map, nextId));
    Op* ret = cloned.back().get();
    if (ret->name != "return" || ret->operands.size() != op->results.size())
      throw CompileError("call @" + callee->name + ": result count mismatch");
    for (size_t q = 0; q < op->results.size(); ++q) repl[op->results[q].get()] = ret->operands[q];
    cloned.pop_back();
    // keep the call op alive (its result Values are referenced by `repl` keys) but mark it dead
    op->dead = true;
    size_t nIns = cloned.size();
    for (auto& c : cloned) c->parent = &r;
    r.ops.insert(r.ops.begin() + k, std::make_move_iterator(cloned.begin()), std::make_move_iterator(cloned.end()));
    // re-scan the inlined ops (they may contain calls themselves)
    any = true;
    k += nIns;  // now points at the dead call
    (void)ret;
  }
  return any;
}

void removeDead(Region& r) {
  for (auto& o : r.ops) for (auto& sub : o->regions) removeDead(*sub);
  std::vector<std::unique_ptr<Op>> keep;
  for (auto& o : r.ops) if (!o->dead) keep.push_back(std::move(o));
  r.ops.swap(keep);
}

void collectUses(const Region& r, std::unordered_map<const Value*, int>& uses) {
  for (auto& o : r.ops) {
    if (o->dead) continue;
    for (auto* v : o->operands) uses[v]++;
    for (auto& sub : o->regions) collectUses(*sub, uses);
  }
}

bool sweep(Region& r, std::unordered_map<const Value*, int>& uses) {
  bool changed = false;
  for (int k = (int)r.ops.size() - 1; k >= 0; --k) {
    Op* o = r.ops[k].get();
    if (o->dead) continue;
    if (o->name != "return") {
      bool used = false;
      for (auto& v : o->results) if (uses[v.get()] > 0) used = true;
      if (!used) {
        o->dead = true;
        std::function<void(Op*)> drop = [&](Op* q) {
          for (auto* v : q->operands) uses[v]--;
          for (auto& sub : q->regions) for (auto& qq : sub->ops) if (!qq->dead) drop(qq.get());
        };
        drop(o);
        changed = true;
        continue;
      }
    }
    for (auto& sub : o->regions) changed |= sweep(*sub, uses);
  }
  return changed;
}

// custom_call @mhlo.asin(%x) and its siblings are the chlo unary ops under another spelling
// (reference: ops/control_flow.cc:53-63, 1417-1440)
void renameUnaryCustomCalls(Region& r) {
  static const std::set<std::string> unary = {"asin", "acos", "atan", "sinh", "cosh", "asinh", "acosh", "atanh", "erf", "erf_inv"};
  for (auto& o : r.ops) {
    for (auto& sub : o->regions) renameUnaryCustomCalls(*sub);
    if (o->name != "custom_call") continue;
    const std::string& t = o->str("target");
    if (t == "mhlo.topk") {
      // the older spelling of chlo.top_k: k is the extent of the results' last dim (reference: ops/control_flow.cc:1461-1477)
      if (o->operands.size() != 1 || o->results.size() != 2) throw CompileError("stablehlo.custom_call mhlo.topk: expected 1 input and 2 outputs");
      const TensorType& vt = o->results[0]->type;
      if (vt.rank() < 1) throw CompileError("stablehlo.custom_call mhlo.topk: the results must have at least one dim");
      Attr k;
      k.kind = Attr::Int;
      k.i = vt.dims.back();
      o->attrs["k"] = k;
      o->name = "chlo.top_k";
      continue;
    }
    if (o->operands.size() != 1 || o->results.size() != 1) continue;
    if (t.rfind("mhlo.", 0) == 0 && unary.count(t.substr(5))) o->name = "chlo." + t.substr(5);
  }
}

}  // namespace

void inlineCalls(Module& m) {
  Func* main = m.main();
  int nextId = 0;
  for (auto& f : m.funcs) nextId = std::max(nextId, maxValueId(f->body) + 1);
  VMap repl;
  for (int iter = 0; iter < 64; ++iter) {
    if (!inlineRegion(m, main->body, repl, nextId, 0)) break;
    applyReplacements(main->body, repl);
    // dead call ops must stay until replacements are resolved, then go
    removeDead(main->body);
    repl.clear();
  }
  renameUnaryCustomCalls(main->body);
}

// ---- integer / boolean dot_general ---------------------------------------------------------
// The matrix cores have no exact 32-bit integer mode, and integer contractions are rare and
// small on this path, so they are rewritten into ops the fused-reduction generator already
// handles exactly:  broadcast both operands to [batch..., lhs free..., rhs free..., contracting...],
// multiply (and for i1), reduce with add (or for i1) over the trailing dims.  Wrap-around
// arithmetic, no detour through floats (the reference round-trips through f32 and is exact
// only below 2^24: ops/linalg.cc:196-250).
namespace {

Value* addResult(Op* op, const TensorType& t, int& nextId) {
  auto v = std::make_unique<Value>();
  v->id = nextId++;
  v->type = t;
  v->def = op;
  v->defIndex = (int)op->results.size();
  v->name = "%lowered" + std::to_string(v->id);
  op->results.push_back(std::move(v));
  return op->results.back().get();
}

std::unique_ptr<Op> makeOp(const std::string& name, std::vector<Value*> operands, Region* parent, int line) {
  auto op = std::make_unique<Op>();
  op->name = name;
  op->operands = std::move(operands);
  op->parent = parent;
  op->line = line;
  return op;
}

Attr intsAttr(const std::vector<int64_t>& v) {
  Attr a;
  a.kind = Attr::Ints;
  a.ints = v;
  return a;
}

void lowerIntegerDotsIn(Region& r, int& nextId) {
  for (size_t k = 0; k < r.ops.size(); ++k) {
    Op* op = r.ops[k].get();
    for (auto& sub : op->regions) lowerIntegerDotsIn(*sub, nextId);
    if (op->name != "dot_general" && op->name != "dot") continue;
    Value* a = op->operands[0];
    Value* b = op->operands[1];
    if (isFloat(a->type.dt)) continue;
    Value* c = op->result();
    const DType et = c->type.dt;
    const bool pred = et == DType::Pred;
    std::vector<int64_t> ab = op->ints("lhs_batch"), bb = op->ints("rhs_batch"), ac = op->ints("lhs_contract"), bc = op->ints("rhs_contract");
    if (op->name == "dot") { ac = {a->type.rank() - 1}; bc = {0}; }
    auto has = [](const std::vector<int64_t>& v, int64_t x) { return std::find(v.begin(), v.end(), x) != v.end(); };
    std::vector<int64_t> af, bf;
    for (int d = 0; d < a->type.rank(); ++d) if (!has(ab, d) && !has(ac, d)) af.push_back(d);
    for (int d = 0; d < b->type.rank(); ++d) if (!has(bb, d) && !has(bc, d)) bf.push_back(d);
    // the common index space and where each operand dim sits in it
    std::vector<int64_t> space, aMap(a->type.rank()), bMap(b->type.rank());
    for (size_t q = 0; q < ab.size(); ++q) { aMap[ab[q]] = (int64_t)space.size(); bMap[bb[q]] = (int64_t)space.size(); space.push_back(a->type.dims[ab[q]]); }
    for (auto d : af) { aMap[d] = (int64_t)space.size(); space.push_back(a->type.dims[d]); }
    for (auto d : bf) { bMap[d] = (int64_t)space.size(); space.push_back(b->type.dims[d]); }
    std::vector<int64_t> redDims;
    for (size_t q = 0; q < ac.size(); ++q) {
      aMap[ac[q]] = (int64_t)space.size(); bMap[bc[q]] = (int64_t)space.size();
      redDims.push_back((int64_t)space.size());
      space.push_back(a->type.dims[ac[q]]);
    }
    std::vector<std::unique_ptr<Op>> made;
    auto emit = [&](std::unique_ptr<Op> o, const TensorType& t) { Value* v = addResult(o.get(), t, nextId); made.push_back(std::move(o)); return v; };
    auto widen = [&](Value* v) {   // operands take the result's element type first (preferred_element_type)
      if (v->type.dt == et) return v;
      TensorType t = v->type;
      t.dt = et;
      return emit(makeOp("convert", {v}, &r, op->line), t);
    };
    TensorType st;
    st.dt = et;
    st.dims = space;
    auto spread = [&](Value* v, const std::vector<int64_t>& map) {
      auto o = makeOp("broadcast_in_dim", {v}, &r, op->line);
      o->attrs["dims"] = intsAttr(map);
      return emit(std::move(o), st);
    };
    Value* A = spread(widen(a), aMap);
    Value* B = spread(widen(b), bMap);
    Value* prod = emit(makeOp(pred ? "and" : "multiply", {A, B}, &r, op->line), st);
    // init: zero of the element type
    auto zero = makeOp("constant", {}, &r, op->line);
    Attr dv;
    dv.kind = Attr::Dense;
    dv.dense = std::make_shared<DenseData>();
    dv.dense->type.dt = et;
    dv.dense->splat = true;
    dv.dense->bytes.assign(dtypeSize(et), 0);
    zero->attrs["value"] = dv;
    TensorType scalar;
    scalar.dt = et;
    Value* z = emit(std::move(zero), scalar);
    // the reduce takes over the dot's result value, so its users need no rewiring
    auto red = makeOp("reduce", {prod, z}, &r, op->line);
    red->attrs["dimensions"] = intsAttr(redDims);
    auto body = std::make_unique<Region>();
    body->parent = red.get();
    for (int q = 0; q < 2; ++q) {
      auto arg = std::make_unique<Value>();
      arg->id = nextId++;
      arg->type = scalar;
      arg->argOf = body.get();
      arg->defIndex = q;
      arg->name = "%lowered_arg" + std::to_string(arg->id);
      body->args.push_back(std::move(arg));
    }
    auto comb = makeOp(pred ? "or" : "add", {body->args[0].get(), body->args[1].get()}, body.get(), op->line);
    Value* cv = addResult(comb.get(), scalar, nextId);
    auto ret = makeOp("return", {cv}, body.get(), op->line);
    body->ops.push_back(std::move(comb));
    body->ops.push_back(std::move(ret));
    red->regions.push_back(std::move(body));
    red->results = std::move(op->results);
    for (auto& v : red->results) v->def = red.get();
    if (redDims.empty()) {
      // nothing to contract: the product is the result
      red->name = "reshape";
      red->operands = {prod};
      red->regions.clear();
      red->attrs.clear();
    }
    made.push_back(std::move(red));
    size_t nIns = made.size();
    r.ops.erase(r.ops.begin() + k);
    r.ops.insert(r.ops.begin() + k, std::make_move_iterator(made.begin()), std::make_move_iterator(made.end()));
    k += nIns - 1;
  }
}

}  // namespace

void lowerIntegerDots(Module& m) {
  Func* f = m.main();
  if (!f) return;
  int nextId = maxValueId(f->body) + 1;
  lowerIntegerDotsIn(f->body, nextId);
}

// ---- general scatter -------------------------------------------------------------------------
// A scatter that is not "whole rows along dim 0" is rewritten into that form over single
// elements: every update element gets the linear index of the operand element it lands on
// (computed with iota / slice / broadcast / multiply-add, i.e. one fused kernel), or an
// out-of-range key when its window does not fit the operand; the flattened operand is then
// scattered one element per "row".  The ordered fold of the row scatter therefore gives the
// sequential update order for every scatter form (reference: DetectScatterType / ApplyScatter,
// ops/gather_scatter.cc:296-699, which leaves the order to float atomics).
namespace {

bool isRowScatter(const Op& op) {
  if (op.operands.size() != 3) return false;
  const TensorType& operand = op.operands[0]->type;
  const TensorType& idx = op.operands[1]->type;
  const TensorType& upd = op.operands[2]->type;
  auto& uwd = op.ints("update_window_dims");
  if (operand.rank() < 1 || op.ints("inserted_window_dims") != std::vector<int64_t>{0} ||
      op.ints("scatter_dims_to_operand_dims") != std::vector<int64_t>{0} || !op.ints("input_batching_dims").empty())
    return false;
  int nScatter = upd.rank() - (int)uwd.size();
  for (size_t k = 0; k < uwd.size(); ++k) if (uwd[k] != nScatter + (int64_t)k) return false;
  if ((int)uwd.size() != operand.rank() - 1) return false;
  for (size_t k = 0; k < uwd.size(); ++k) if (upd.dims[uwd[k]] != operand.dims[1 + k]) return false;
  int64_t nUpd = 1;
  for (int d = 0; d < nScatter; ++d) nUpd *= upd.dims[d];
  int64_t ivd = op.integer("index_vector_dim");
  if (ivd < idx.rank() && idx.dims[ivd] != 1) return false;
  return idx.numel() == nUpd;
}

void lowerScattersIn(Region& r, int& nextId) {
  for (size_t k = 0; k < r.ops.size(); ++k) {
    Op* op = r.ops[k].get();
    for (auto& sub : op->regions) lowerScattersIn(*sub, nextId);
    if (op->name != "scatter" || op->operands.size() != 3 || isRowScatter(*op)) continue;
    Value* operand = op->operands[0];
    Value* idx = op->operands[1];
    Value* upd = op->operands[2];
    const TensorType ot = operand->type, it = idx->type, ut = upd->type;
    const int64_t P = ot.numel(), n = ut.numel();
    if (P >= (int64_t(1) << 32) - 1) throw CompileError("stablehlo.scatter: operand too large for element-wise lowering");
    auto uwd = op->ints("update_window_dims"), iwd = op->ints("inserted_window_dims"), ibd = op->ints("input_batching_dims"),
         sibd = op->ints("scatter_indices_batching_dims"), sdo = op->ints("scatter_dims_to_operand_dims");
    const int64_t ivd = op->has("index_vector_dim") ? op->integer("index_vector_dim") : it.rank();
    auto has = [](const std::vector<int64_t>& v, int64_t x) { return std::find(v.begin(), v.end(), x) != v.end(); };
    std::vector<int64_t> sd;                       // scatter dims of the updates, in order
    for (int d = 0; d < ut.rank(); ++d) if (!has(uwd, d)) sd.push_back(d);
    std::vector<int64_t> idxBatchAxes;             // dims of the index tensor except the vector dim
    for (int d = 0; d < it.rank(); ++d) if (d != ivd) idxBatchAxes.push_back(d);
    if (idxBatchAxes.size() != sd.size()) throw CompileError("stablehlo.scatter: index and update ranks do not agree");
    std::vector<int64_t> winDims;                  // operand dims that carry a window coordinate
    for (int d = 0; d < ot.rank(); ++d) if (!has(iwd, d) && !has(ibd, d)) winDims.push_back(d);
    if (winDims.size() != uwd.size()) throw CompileError("stablehlo.scatter: update_window_dims do not match the operand");

    std::vector<std::unique_ptr<Op>> made;
    auto emit = [&](std::unique_ptr<Op> o, const TensorType& t) { Value* v = addResult(o.get(), t, nextId); made.push_back(std::move(o)); return v; };
    TensorType i64u;                // int64 over the update index space
    i64u.dt = DType::S64;
    i64u.dims = ut.dims;
    TensorType predu = i64u;
    predu.dt = DType::Pred;
    auto splat = [&](int64_t x) {
      auto c = makeOp("constant", {}, &r, op->line);
      Attr dv;
      dv.kind = Attr::Dense;
      dv.dense = std::make_shared<DenseData>();
      dv.dense->type.dt = DType::S64;
      dv.dense->type.dims = ut.dims;
      dv.dense->splat = true;
      dv.dense->bytes.resize(8);
      memcpy(dv.dense->bytes.data(), &x, 8);
      c->attrs["value"] = dv;
      return emit(std::move(c), i64u);
    };
    auto iota = [&](int64_t dim) {
      auto o = makeOp("iota", {}, &r, op->line);
      Attr a;
      a.kind = Attr::Int;
      a.i = dim;
      o->attrs["dim"] = a;
      return emit(std::move(o), i64u);
    };
    auto binary = [&](const char* name, Value* a, Value* b, const TensorType& t) { return emit(makeOp(name, {a, b}, &r, op->line), t); };
    auto compare = [&](const char* dir, Value* a, Value* b) {
      auto o = makeOp("compare", {a, b}, &r, op->line);
      Attr d;
      d.kind = Attr::Str;
      d.s = dir;
      o->attrs["direction"] = d;
      return emit(std::move(o), predu);
    };
    // component q of the index vector, spread over the update index space
    auto component = [&](int64_t q) {
      Value* v = idx;
      if (ivd < it.rank()) {
        auto sl = makeOp("slice", {idx}, &r, op->line);
        std::vector<int64_t> st(it.rank(), 0), lim = it.dims, sr(it.rank(), 1);
        st[ivd] = q;
        lim[ivd] = q + 1;
        sl->attrs["start"] = intsAttr(st);
        sl->attrs["limit"] = intsAttr(lim);
        sl->attrs["strides"] = intsAttr(sr);
        TensorType t = it;
        t.dims[ivd] = 1;
        v = emit(std::move(sl), t);
      }
      TensorType bt;
      bt.dt = it.dt;
      for (auto a : idxBatchAxes) bt.dims.push_back(it.dims[a]);
      v = emit(makeOp("reshape", {v}, &r, op->line), bt);
      TensorType ct = bt;
      ct.dt = DType::S64;
      if (bt.dt != DType::S64) v = emit(makeOp("convert", {v}, &r, op->line), ct);
      auto bc = makeOp("broadcast_in_dim", {v}, &r, op->line);
      bc->attrs["dims"] = intsAttr(sd);
      return emit(std::move(bc), i64u);
    };
    std::vector<int64_t> stride(ot.rank(), 1);
    for (int d = ot.rank() - 2; d >= 0; --d) stride[d] = stride[d + 1] * ot.dims[d + 1];
    Value* lin = splat(0);
    Value* inb = nullptr;
    for (int d = 0; d < ot.rank(); ++d) {
      Value* coord = nullptr;
      auto add = [&](Value* v) { coord = coord ? binary("add", coord, v, i64u) : v; };
      auto sIt = std::find(sdo.begin(), sdo.end(), (int64_t)d);
      int64_t ws = 1;
      auto wIt = std::find(winDims.begin(), winDims.end(), (int64_t)d);
      if (wIt != winDims.end()) ws = ut.dims[uwd[wIt - winDims.begin()]];
      if (sIt != sdo.end()) {
        Value* start = component(sIt - sdo.begin());
        Value* ok = binary("and", compare("GE", start, splat(0)), compare("LE", start, splat(ot.dims[d] - ws)), predu);
        inb = inb ? binary("and", inb, ok, predu) : ok;
        add(start);
      }
      if (wIt != winDims.end()) add(iota(uwd[wIt - winDims.begin()]));
      auto bIt = std::find(ibd.begin(), ibd.end(), (int64_t)d);
      if (bIt != ibd.end()) {
        int64_t ib = sibd.at(bIt - ibd.begin());
        auto pos = std::find(idxBatchAxes.begin(), idxBatchAxes.end(), ib);
        if (pos == idxBatchAxes.end()) throw CompileError("stablehlo.scatter: scatter_indices_batching_dims names the index vector dim");
        add(iota(sd[pos - idxBatchAxes.begin()]));
      }
      if (!coord) continue;
      lin = binary("add", lin, stride[d] == 1 ? coord : binary("multiply", coord, splat(stride[d]), i64u), i64u);
    }
    Value* key64 = lin;
    if (inb) {
      auto sel = makeOp("select", {inb, lin, splat(P)}, &r, op->line);
      key64 = emit(std::move(sel), i64u);
    }
    TensorType keyT = i64u;
    keyT.dt = DType::U32;
    Value* key = emit(makeOp("convert", {key64}, &r, op->line), keyT);
    TensorType flatKey;
    flatKey.dt = DType::U32;
    flatKey.dims = {n};
    key = emit(makeOp("reshape", {key}, &r, op->line), flatKey);
    TensorType flatUpd;
    flatUpd.dt = ut.dt;
    flatUpd.dims = {n};
    Value* fu = emit(makeOp("reshape", {upd}, &r, op->line), flatUpd);
    TensorType flatOp;
    flatOp.dt = ot.dt;
    flatOp.dims = {P};
    Value* fo = emit(makeOp("reshape", {operand}, &r, op->line), flatOp);
    // the element scatter keeps the original body
    auto sc = makeOp("scatter", {fo, key, fu}, &r, op->line);
    sc->attrs["update_window_dims"] = intsAttr({});
    sc->attrs["inserted_window_dims"] = intsAttr({0});
    sc->attrs["scatter_dims_to_operand_dims"] = intsAttr({0});
    Attr one;
    one.kind = Attr::Int;
    one.i = 1;
    sc->attrs["index_vector_dim"] = one;
    for (auto& kv : op->attrs)
      if (kv.first == "unique_indices" || kv.first == "indices_are_sorted") sc->attrs[kv.first] = kv.second;
    sc->regions = std::move(op->regions);
    for (auto& rg : sc->regions) rg->parent = sc.get();
    Value* flatRes = emit(std::move(sc), flatOp);
    // a reshape takes over the original result value
    auto back = makeOp("reshape", {flatRes}, &r, op->line);
    back->results = std::move(op->results);
    for (auto& v : back->results) v->def = back.get();
    made.push_back(std::move(back));
    size_t nIns = made.size();
    r.ops.erase(r.ops.begin() + k);
    r.ops.insert(r.ops.begin() + k, std::make_move_iterator(made.begin()), std::make_move_iterator(made.end()));
    k += nIns - 1;
  }
}

}  // namespace

// ---- reduce_window / select_and_scatter (pooling) ----------------------------------------------
// A window reduction with a small window is the combination of one strided slice of the padded
// operand per window tap; the rewrite emits exactly that (pad, k slices, k-1 combiner ops) and
// the fusion planner turns it back into a single kernel whose index arithmetic walks the
// window.  select_and_scatter (the gradient of max pooling) becomes: find the selected tap of
// every window with a running compare over the same slices (first occurrence wins, as the
// sequential definition does), then add, per tap, the source values whose window selected
// that tap, dilated by the stride and shifted into operand coordinates with a pad.
// (reference: ops/reduction.cc:165-626 pooling tier.)
namespace {

std::vector<int64_t> denseInts(const Attr& a, size_t n) {
  std::vector<int64_t> out(n, 0);
  if (a.kind == Attr::Ints) { for (size_t i = 0; i < n && i < a.ints.size(); ++i) out[i] = a.ints[i]; return out; }
  if (a.kind != Attr::Dense || !a.dense) return out;
  const DenseData& d = *a.dense;
  size_t esz = dtypeSize(d.type.dt);
  for (size_t i = 0; i < n; ++i) {
    const uint8_t* p = d.bytes.data() + (d.splat ? 0 : i * esz);
    if ((d.splat ? esz : (i + 1) * esz) > d.bytes.size()) break;
    int64_t v = 0;
    if (esz == 8) memcpy(&v, p, 8);
    else if (esz == 4) { int32_t t; memcpy(&t, p, 4); v = t; }
    else if (esz == 1) v = (int8_t)p[0];
    out[i] = v;
  }
  return out;
}

// name of the single binary op a two-argument region applies to its arguments, or ""
std::string regionBinaryOp(const Region& r) {
  if (r.args.size() != 2 || r.ops.size() != 2) return "";
  Op* b = r.ops[0].get();
  Op* ret = r.ops[1].get();
  if (ret->name != "return" || ret->operands.size() != 1 || ret->operands[0] != b->result() || b->operands.size() != 2) return "";
  bool uses = (b->operands[0] == r.args[0].get() && b->operands[1] == r.args[1].get()) ||
              (b->operands[0] == r.args[1].get() && b->operands[1] == r.args[0].get());
  return uses ? b->name : "";
}

struct WindowSpec {
  int rank = 0;
  std::vector<int64_t> size, stride, baseDil, winDil, padLo, padHi;
  int64_t taps = 1;
};

WindowSpec windowSpec(const Op& op, int rank) {
  WindowSpec w;
  w.rank = rank;
  auto get = [&](const char* name, int64_t dflt) {
    std::vector<int64_t> v(rank, dflt);
    auto it = op.attrs.find(name);
    if (it != op.attrs.end()) { auto x = denseInts(it->second, rank); if (!it->second.ints.empty() || it->second.kind == Attr::Dense) v = x; }
    return v;
  };
  w.size = get("window_dimensions", 1);
  w.stride = get("window_strides", 1);
  w.baseDil = get("base_dilations", 1);
  w.winDil = get("window_dilations", 1);
  w.padLo.assign(rank, 0);
  w.padHi.assign(rank, 0);
  auto it = op.attrs.find("padding");
  if (it != op.attrs.end()) {
    auto p = denseInts(it->second, 2 * (size_t)rank);
    for (int d = 0; d < rank; ++d) { w.padLo[d] = p[2 * d]; w.padHi[d] = p[2 * d + 1]; }
  }
  for (auto k : w.size) w.taps *= k;
  return w;
}

struct Rewriter {
  Region& r;
  int& nextId;
  int line;
  std::vector<std::unique_ptr<Op>> made;
  Value* emit(std::unique_ptr<Op> o, const TensorType& t) { Value* v = addResult(o.get(), t, nextId); made.push_back(std::move(o)); return v; }
  Value* unary(const char* name, Value* a, const TensorType& t) { return emit(makeOp(name, {a}, &r, line), t); }
  Value* binary(const std::string& name, Value* a, Value* b, const TensorType& t) { return emit(makeOp(name, {a, b}, &r, line), t); }
  Value* broadcastScalar(Value* s, const TensorType& t) {
    auto o = makeOp("broadcast_in_dim", {s}, &r, line);
    o->attrs["dims"] = intsAttr({});
    return emit(std::move(o), t);
  }
  Value* pad(Value* x, Value* padValue, const std::vector<int64_t>& lo, const std::vector<int64_t>& hi, const std::vector<int64_t>& interior) {
    bool trivial = true;
    TensorType t = x->type;
    for (int d = 0; d < t.rank(); ++d) {
      if (lo[d] || hi[d] || interior[d]) trivial = false;
      t.dims[d] = std::max<int64_t>(0, (x->type.dims[d] > 0 ? (x->type.dims[d] - 1) * (interior[d] + 1) + 1 : 0) + lo[d] + hi[d]);
    }
    if (trivial) return x;
    auto o = makeOp("pad", {x, padValue}, &r, line);
    o->attrs["low"] = intsAttr(lo);
    o->attrs["high"] = intsAttr(hi);
    o->attrs["interior"] = intsAttr(interior);
    return emit(std::move(o), t);
  }
  Value* slice(Value* x, const std::vector<int64_t>& start, const std::vector<int64_t>& count, const std::vector<int64_t>& stride) {
    TensorType t = x->type;
    std::vector<int64_t> limit(start.size());
    bool whole = true;
    for (size_t d = 0; d < start.size(); ++d) {
      t.dims[d] = count[d];
      limit[d] = start[d] + (count[d] > 0 ? (count[d] - 1) * stride[d] + 1 : 0);
      if (start[d] != 0 || stride[d] != 1 || count[d] != x->type.dims[d]) whole = false;
    }
    if (whole) return x;
    auto o = makeOp("slice", {x}, &r, line);
    o->attrs["start"] = intsAttr(start);
    o->attrs["limit"] = intsAttr(limit);
    o->attrs["strides"] = intsAttr(stride);
    return emit(std::move(o), t);
  }
  Value* splat(DType dt, const std::vector<int64_t>& dims, const void* bytes) {
    auto c = makeOp("constant", {}, &r, line);
    Attr dv;
    dv.kind = Attr::Dense;
    dv.dense = std::make_shared<DenseData>();
    dv.dense->type.dt = dt;
    dv.dense->type.dims = dims;
    dv.dense->splat = true;
    dv.dense->bytes.assign((const uint8_t*)bytes, (const uint8_t*)bytes + dtypeSize(dt));
    c->attrs["value"] = dv;
    TensorType t;
    t.dt = dt;
    t.dims = dims;
    return emit(std::move(c), t);
  }
  // replaces op k of the region by the ops made so far; `last` takes over the results of the replaced op
  void finish(size_t& k, Op* replaced, std::unique_ptr<Op> last) {
    last->results = std::move(replaced->results);
    for (auto& v : last->results) v->def = last.get();
    made.push_back(std::move(last));
    size_t nIns = made.size();
    r.ops.erase(r.ops.begin() + k);
    r.ops.insert(r.ops.begin() + k, std::make_move_iterator(made.begin()), std::make_move_iterator(made.end()));
    k += nIns - 1;
    made.clear();
  }
};

constexpr int64_t kMaxWindowTaps = 64;

// the slices of the padded operand, one per window tap in row-major tap order
std::vector<Value*> tapSlices(Rewriter& rw, Value* padded, const WindowSpec& w, const std::vector<int64_t>& outDims) {
  std::vector<Value*> taps;
  std::vector<int64_t> t(w.rank, 0);
  for (int64_t n = 0; n < w.taps; ++n) {
    std::vector<int64_t> start(w.rank);
    for (int d = 0; d < w.rank; ++d) start[d] = t[d] * w.winDil[d];
    taps.push_back(rw.slice(padded, start, outDims, w.stride));
    for (int d = w.rank - 1; d >= 0; --d) { if (++t[d] < w.size[d]) break; t[d] = 0; }
  }
  return taps;
}

// whether `init` is a constant holding the identity of the reducer `comb` for its element type
bool isReducerIdentity(Value* init, const std::string& comb) {
  Op* d = init->def;
  while (d && (d->name == "broadcast_in_dim" || d->name == "reshape") && d->operands.size() == 1) d = d->operands[0]->def;
  if (!d || d->name != "constant" || !d->has("value") || !d->attrs.at("value").dense) return false;
  const DenseData& dd = *d->attrs.at("value").dense;
  if (!dd.splat && dd.type.numel() != 1) return false;
  const DType dt = dd.type.dt;
  const size_t sz = dtypeSize(dt);
  if (dd.bytes.size() < sz) return false;
  if (isFloat(dt)) {
    double v;
    if (dt == DType::F32) { float f; memcpy(&f, dd.bytes.data(), 4); v = f; }
    else if (dt == DType::F64) memcpy(&v, dd.bytes.data(), 8);
    else if (dt == DType::BF16) { uint16_t h; memcpy(&h, dd.bytes.data(), 2); uint32_t u = (uint32_t)h << 16; float f; memcpy(&f, &u, 4); v = f; }
    else if (dt == DType::F16) { _Float16 h; memcpy(&h, dd.bytes.data(), 2); v = (double)(float)h; }
    else return false;
    if (comb == "add") return v == 0.0;
    if (comb == "multiply") return v == 1.0;
    if (comb == "maximum") return v == -__builtin_inf();
    if (comb == "minimum") return v == __builtin_inf();
    return false;
  }
  uint64_t bits = 0;
  memcpy(&bits, dd.bytes.data(), sz);
  const uint64_t ones = sz == 8 ? ~0ull : ((1ull << (8 * sz)) - 1);
  const bool sg = dt == DType::S8 || dt == DType::S16 || dt == DType::S32 || dt == DType::S64;
  if (dt == DType::Pred) {
    const bool b = dd.bytes[0] != 0;
    return (comb == "add" || comb == "or" || comb == "xor" || comb == "maximum") ? !b : b;   // multiply, and, minimum: true
  }
  if (comb == "add" || comb == "or" || comb == "xor") return bits == 0;
  if (comb == "multiply") return bits == 1;
  if (comb == "and") return bits == ones;
  if (comb == "maximum") return bits == (sg ? (1ull << (8 * sz - 1)) : 0ull);
  if (comb == "minimum") return bits == (sg ? (ones >> 1) : ones);
  return false;
}

void lowerWindowOpsIn(Region& r, int& nextId) {
  for (size_t k = 0; k < r.ops.size(); ++k) {
    Op* op = r.ops[k].get();
    for (auto& sub : op->regions) lowerWindowOpsIn(*sub, nextId);
    if (op->name == "reduce_window") {
      if (op->operands.size() != 2 || op->regions.size() != 1) throw CompileError("stablehlo.reduce_window with several inputs is not supported");
      Value* x = op->operands[0];
      Value* init = op->operands[1];
      const TensorType rt = op->result()->type;
      std::string comb = regionBinaryOp(*op->regions[0]);
      static const std::set<std::string> ok = {"add", "multiply", "maximum", "minimum", "and", "or", "xor"};
      if (!ok.count(comb)) throw CompileError("stablehlo.reduce_window: the reducer must be a single add / multiply / maximum / minimum / and / or / xor");
      WindowSpec w = windowSpec(*op, x->type.rank());
      Rewriter rw{r, nextId, op->line, {}};
      if (w.taps > kMaxWindowTaps) {
        // Cumulative pattern (cumsum / cumprod / cummax as JAX lowers them): the window spans one whole
        // dim, padded by n-1 on one side.  Computed as a Hillis-Steele scan: log2(n) passes of
        // "combine with a copy of yourself shifted by s", each pass kept in memory.
        int axis = -1;
        bool cumulative = true;
        for (int d = 0; d < w.rank; ++d) {
          if (w.stride[d] != 1 || w.baseDil[d] != 1 || w.winDil[d] != 1) cumulative = false;
          if (w.size[d] == 1) { if (w.padLo[d] || w.padHi[d]) cumulative = false; continue; }
          if (axis >= 0 || w.size[d] != x->type.dims[d]) cumulative = false;
          axis = d;
        }
        const int64_t n = axis >= 0 ? x->type.dims[axis] : 0;
        const bool forward = cumulative && axis >= 0 && w.padLo[axis] == n - 1 && w.padHi[axis] == 0;
        const bool backward = cumulative && axis >= 0 && w.padLo[axis] == 0 && w.padHi[axis] == n - 1;
        if (!forward && !backward) {
          // A rectangular window is the product of one window per dim, and the reducers taken here are associative
          // and commutative: reduce dim after dim (14 + 14 taps for a 14 x 14 pooling window instead of 196).  Padding
          // cells hold the init value, which has to be the reducer's identity for the stages to compose.
          bool perDim = isReducerIdentity(init, comb);
          for (int d = 0; d < w.rank; ++d) if (w.size[d] > kMaxWindowTaps) perDim = false;
          if (!perDim)
            throw CompileError("stablehlo.reduce_window: windows of more than 64 elements need the reducer's identity as init value and at most 64 elements per dim "
                               "(or the cumulative form: one whole dim, padded by n-1 on one side)");
          Value* cur = x;
          std::vector<int> stages;
          for (int d = 0; d < w.rank; ++d)
            if (w.size[d] != 1 || w.stride[d] != 1 || w.padLo[d] || w.padHi[d] || w.baseDil[d] != 1) stages.push_back(d);
          for (size_t q = 0; q < stages.size(); ++q) {
            const int d = stages[q];
            WindowSpec one;
            one.rank = w.rank;
            one.size.assign(w.rank, 1); one.stride.assign(w.rank, 1); one.baseDil.assign(w.rank, 1); one.winDil.assign(w.rank, 1);
            one.padLo.assign(w.rank, 0); one.padHi.assign(w.rank, 0);
            one.size[d] = w.size[d]; one.stride[d] = w.stride[d]; one.winDil[d] = w.winDil[d];
            one.taps = w.size[d];
            std::vector<int64_t> lo(w.rank, 0), hi(w.rank, 0), interior(w.rank, 0);
            lo[d] = w.padLo[d]; hi[d] = w.padHi[d]; interior[d] = w.baseDil[d] - 1;
            Value* padded = rw.pad(cur, init, lo, hi, interior);
            TensorType st = cur->type;
            st.dims[d] = rt.dims[d];
            auto taps = tapSlices(rw, padded, one, st.dims);
            const bool lastStage = q + 1 == stages.size();
            Value* acc = taps[0];
            for (size_t t = 1; t < taps.size(); ++t) {
              if (lastStage && t + 1 == taps.size()) break;
              acc = rw.binary(comb, acc, taps[t], st);
            }
            if (lastStage) {
              // (a last stage of one tap still needs an op to carry the results: the identity combined with it)
              auto last = taps.size() == 1 ? makeOp(comb, {rw.broadcastScalar(init, st), acc}, &r, op->line) : makeOp(comb, {acc, taps.back()}, &r, op->line);
              rw.finish(k, op, std::move(last));
            } else {
              cur = acc;
            }
          }
          continue;
        }
        Value* cur = x;
        std::vector<int64_t> zeros(w.rank, 0);
        for (int64_t sft = 1; sft < n; sft *= 2) {
          std::vector<int64_t> lo = zeros, hi = zeros;
          lo[axis] = forward ? sft : -sft;
          hi[axis] = forward ? -sft : sft;
          Value* shifted = rw.pad(cur, init, lo, hi, zeros);
          auto step = makeOp(comb, {cur, shifted}, &r, op->line);
          Attr flag;
          flag.kind = Attr::Bool;
          flag.b = true;
          step->attrs["force_materialize"] = flag;   // each pass reads the previous one at two places: recomputing it would double the work per pass
          cur = rw.emit(std::move(step), rt);
        }
        auto last = makeOp(comb, {rw.broadcastScalar(init, rt), cur}, &r, op->line);
        rw.finish(k, op, std::move(last));
        continue;
      }
      std::vector<int64_t> interior(w.rank);
      for (int d = 0; d < w.rank; ++d) interior[d] = w.baseDil[d] - 1;
      Value* padded = rw.pad(x, init, w.padLo, w.padHi, interior);
      auto taps = tapSlices(rw, padded, w, rt.dims);
      Value* acc = rw.broadcastScalar(init, rt);
      for (size_t t = 0; t + 1 < taps.size() + 1 && t < taps.size(); ++t) {
        if (t + 1 == taps.size()) break;
        acc = rw.binary(comb, acc, taps[t], rt);
      }
      auto last = makeOp(comb, {acc, taps.back()}, &r, op->line);
      rw.finish(k, op, std::move(last));
      continue;
    }
    if (op->name == "select_and_scatter") {
      if (op->operands.size() != 3 || op->regions.size() != 2) throw CompileError("stablehlo.select_and_scatter: malformed");
      Value* x = op->operands[0];
      Value* src = op->operands[1];
      Value* init = op->operands[2];
      const TensorType rt = op->result()->type;
      if (!isFloat(x->type.dt)) throw CompileError("stablehlo.select_and_scatter: only floating-point operands are supported");
      // select region: one compare of its two arguments
      Region& sel = *op->regions[0];
      std::string dir;
      if (sel.args.size() == 2 && sel.ops.size() == 2 && sel.ops[0]->name == "compare" && sel.ops[0]->operands.size() == 2 &&
          sel.ops[0]->operands[0] == sel.args[0].get() && sel.ops[0]->operands[1] == sel.args[1].get() && sel.ops[1]->name == "return" &&
          sel.ops[1]->operands.size() == 1 && sel.ops[1]->operands[0] == sel.ops[0]->result())
        dir = sel.ops[0]->str("direction");
      if (dir != "GE" && dir != "GT" && dir != "LE" && dir != "LT") throw CompileError("stablehlo.select_and_scatter: the select region must be one GE / GT / LE / LT compare");
      if (regionBinaryOp(*op->regions[1]) != "add") throw CompileError("stablehlo.select_and_scatter: the scatter region must be an add");
      WindowSpec w = windowSpec(*op, x->type.rank());
      if (w.taps > kMaxWindowTaps) throw CompileError("stablehlo.select_and_scatter: windows of more than 64 elements are not supported");
      for (int d = 0; d < w.rank; ++d) if (w.baseDil[d] != 1 || w.winDil[d] != 1) throw CompileError("stablehlo.select_and_scatter: dilations are not supported");
      Rewriter rw{r, nextId, op->line, {}};
      // padding never wins the selection
      const bool wantsLarge = dir == "GE" || dir == "GT";
      float losingF = wantsLarge ? -__builtin_inff() : __builtin_inff();
      uint16_t losingBf = wantsLarge ? 0xFF80 : 0x7F80;
      uint16_t losingH = wantsLarge ? 0xFC00 : 0x7C00;
      double losingD = wantsLarge ? -__builtin_inf() : __builtin_inf();
      const void* lp = x->type.dt == DType::F32 ? (const void*)&losingF : x->type.dt == DType::BF16 ? (const void*)&losingBf
                       : x->type.dt == DType::F16 ? (const void*)&losingH : (const void*)&losingD;
      Value* losing = rw.splat(x->type.dt, {}, lp);
      std::vector<int64_t> zeros(w.rank, 0);
      Value* padded = rw.pad(x, losing, w.padLo, w.padHi, zeros);
      auto taps = tapSlices(rw, padded, w, src->type.dims);
      // running selection over the taps: select(best, candidate) false -> the candidate takes over
      TensorType idxT = src->type;
      idxT.dt = DType::S32;
      TensorType predT = src->type;
      predT.dt = DType::Pred;
      int32_t zero32 = 0;
      Value* bestVal = taps[0];
      Value* bestIdx = rw.splat(DType::S32, src->type.dims, &zero32);
      for (size_t t = 1; t < taps.size(); ++t) {
        auto cmp = makeOp("compare", {bestVal, taps[t]}, &r, op->line);
        Attr d;
        d.kind = Attr::Str;
        d.s = dir;
        cmp->attrs["direction"] = d;
        Value* keep = rw.emit(std::move(cmp), predT);
        int32_t ti = (int32_t)t;
        Value* tv = rw.splat(DType::S32, src->type.dims, &ti);
        bestVal = rw.emit(makeOp("select", {keep, bestVal, taps[t]}, &r, op->line), src->type.dt == x->type.dt ? taps[t]->type : taps[t]->type);
        bestIdx = rw.emit(makeOp("select", {keep, bestIdx, tv}, &r, op->line), idxT);
      }
      // per tap: the sources whose window selected it, moved to operand coordinates
      uint64_t zeroBits = 0;
      Value* zeroScalar = rw.splat(src->type.dt, {}, &zeroBits);
      Value* zeroSrc = rw.splat(src->type.dt, src->type.dims, &zeroBits);
      Value* acc = rw.broadcastScalar(init, rt);
      std::vector<int64_t> t(w.rank, 0), interior(w.rank);
      for (int d = 0; d < w.rank; ++d) interior[d] = w.stride[d] - 1;
      std::unique_ptr<Op> lastOp;
      for (int64_t n = 0; n < w.taps; ++n) {
        int32_t ti = (int32_t)n;
        Value* tv = rw.splat(DType::S32, src->type.dims, &ti);
        auto eq = makeOp("compare", {bestIdx, tv}, &r, op->line);
        Attr d;
        d.kind = Attr::Str;
        d.s = "EQ";
        eq->attrs["direction"] = d;
        Value* hit = rw.emit(std::move(eq), predT);
        Value* contrib = rw.emit(makeOp("select", {hit, src, zeroSrc}, &r, op->line), src->type);
        std::vector<int64_t> lo(w.rank), hi(w.rank);
        for (int dd = 0; dd < w.rank; ++dd) {
          lo[dd] = t[dd] - w.padLo[dd];
          int64_t span = src->type.dims[dd] > 0 ? (src->type.dims[dd] - 1) * w.stride[dd] + 1 : 0;
          hi[dd] = rt.dims[dd] - span - lo[dd];
        }
        Value* placed = rw.pad(contrib, zeroScalar, lo, hi, interior);
        if (n + 1 < w.taps) acc = rw.binary("add", acc, placed, rt);
        else lastOp = makeOp("add", {acc, placed}, &r, op->line);
        for (int dd = w.rank - 1; dd >= 0; --dd) { if (++t[dd] < w.size[dd]) break; t[dd] = 0; }
      }
      rw.finish(k, op, std::move(lastOp));
      continue;
    }
  }
}


// stablehlo.rng_bit_generator -> plain integer ops.  The bits are implementation-defined by the specification
// (the reference draws them from MLX's generator and says so, src/pjrt_plugin/ops/control_flow.cc:2301-2360); what
// callers rely on is the state rule the reference keeps: state = [key, counter] as ui64[2], the counter grows by
// ceil(output bytes / 16).  Here element i of the output is word 0 (and word 1 for 64-bit types) of
// threefry2x32(key = the two halves of state[0], counter = (i, low half of state[1])), which the planner fuses
// into one kernel like any other integer chain.
void lowerRngIn(Region& r, int& nextId) {
  for (size_t k = 0; k < r.ops.size(); ++k) {
    Op* op = r.ops[k].get();
    for (auto& sub : op->regions) lowerRngIn(*sub, nextId);
    if (op->name != "rng_bit_generator") continue;
    if (op->operands.size() != 1 || op->results.size() != 2) throw CompileError("stablehlo.rng_bit_generator: expected one state operand and two results");
    Value* state = op->operands[0];
    const TensorType st = state->type;
    const TensorType ot = op->results[1]->type;
    if (st.dt != DType::U64 || st.rank() != 1 || st.dims[0] < 2 || !(op->results[0]->type == st))
      throw CompileError("stablehlo.rng_bit_generator: the state must be tensor<Nxui64> with N >= 2, got " + st.str());
    const size_t esz = dtypeSize(ot.dt);
    if (!(isInt(ot.dt) || ot.dt == DType::U8 || ot.dt == DType::U16 || ot.dt == DType::U32 || ot.dt == DType::U64) || ot.numel() >= (int64_t(1) << 32))
      throw CompileError("stablehlo.rng_bit_generator: unsupported output type " + ot.str());
    Rewriter rw{r, nextId, op->line, {}};
    auto ty = [](DType dt, std::vector<int64_t> dims) { TensorType t; t.dt = dt; t.dims = std::move(dims); return t; };
    const int64_t N = st.dims[0];
    // ---- new state: counter (element 1) + ceil(bytes / 16)
    const uint64_t incr = ((uint64_t)ot.numel() * esz + 15) / 16;
    Value* head = rw.slice(state, {0}, {1}, {1});
    Value* ctr = rw.slice(state, {1}, {1}, {1});
    Value* ctrNew = rw.binary("add", ctr, rw.splat(DType::U64, {1}, &incr), ty(DType::U64, {1}));
    std::vector<Value*> parts{head, ctrNew};
    if (N > 2) parts.push_back(rw.slice(state, {2}, {N - 2}, {1}));
    auto cat = makeOp("concatenate", parts, &r, op->line);
    Attr dimA;
    dimA.kind = Attr::Int;
    dimA.i = 0;
    cat->attrs["dim"] = dimA;
    // ---- bits
    const TensorType u32t = ty(DType::U32, ot.dims), u64s = ty(DType::U64, {}), u32s = ty(DType::U32, {});
    auto scalarOf = [&](Value* one) { return rw.unary("reshape", one, u64s); };
    const uint64_t sh32 = 32;
    Value* key64 = scalarOf(head);
    Value* ctr64 = scalarOf(ctr);
    Value* k0s = rw.unary("convert", key64, u32s);
    Value* k1s = rw.unary("convert", rw.binary("shift_right_logical", key64, rw.splat(DType::U64, {}, &sh32), u64s), u32s);
    Value* c1s = rw.unary("convert", ctr64, u32s);
    Value* k0 = rw.broadcastScalar(k0s, u32t);
    Value* k1 = rw.broadcastScalar(k1s, u32t);
    Value* c1 = rw.broadcastScalar(c1s, u32t);
    // element index: iota over the flattened output, reshaped to the output dims
    auto io = makeOp("iota", {}, &r, op->line);
    Attr zero;
    zero.kind = Attr::Int;
    zero.i = 0;
    io->attrs["dim"] = zero;
    Value* flat = rw.emit(std::move(io), ty(DType::U32, {ot.numel()}));
    Value* c0 = ot.rank() == 1 ? flat : rw.unary("reshape", flat, u32t);
    auto cu = [&](uint32_t x) { return rw.splat(DType::U32, ot.dims, &x); };
    auto bin = [&](const char* n, Value* a, Value* b) { return rw.binary(n, a, b, u32t); };
    auto rotl = [&](Value* x, uint32_t rbits) { return bin("or", bin("shift_left", x, cu(rbits)), bin("shift_right_logical", x, cu(32 - rbits))); };
    Value* ks[3] = {k0, k1, bin("xor", bin("xor", k0, k1), cu(0x1BD11BDAu))};
    Value* x0 = bin("add", c0, ks[0]);
    Value* x1 = bin("add", c1, ks[1]);
    static const uint32_t rots[2][4] = {{13, 15, 26, 6}, {17, 29, 16, 24}};
    for (uint32_t blk = 0; blk < 5; ++blk) {
      for (uint32_t rr : rots[blk % 2]) {
        x0 = bin("add", x0, x1);
        x1 = bin("xor", rotl(x1, rr), x0);
      }
      x0 = bin("add", x0, ks[(blk + 1) % 3]);
      x1 = bin("add", bin("add", x1, ks[(blk + 2) % 3]), cu(blk + 1));
    }
    std::unique_ptr<Op> last;
    if (esz == 8) {
      const TensorType u64t = ty(DType::U64, ot.dims);
      Value* lo = rw.unary("convert", x0, u64t);
      Value* hi = rw.binary("shift_left", rw.unary("convert", x1, u64t), rw.splat(DType::U64, ot.dims, &sh32), u64t);
      Value* both = rw.binary("or", lo, hi, u64t);
      last = makeOp(ot.dt == DType::U64 ? "reshape" : "bitcast_convert", {both}, &r, op->line);
    } else {
      last = makeOp(ot.dt == DType::U32 ? "reshape" : (esz == 4 ? "bitcast_convert" : "convert"), {x0}, &r, op->line);
    }
    // the two results move to the two final ops
    cat->results.push_back(std::move(op->results[0]));
    cat->results[0]->def = cat.get();
    last->results.push_back(std::move(op->results[1]));
    last->results[0]->def = last.get();
    rw.made.push_back(std::move(cat));
    rw.made.push_back(std::move(last));
    size_t nIns = rw.made.size();
    r.ops.erase(r.ops.begin() + k);
    r.ops.insert(r.ops.begin() + k, std::make_move_iterator(rw.made.begin()), std::make_move_iterator(rw.made.end()));
    k += nIns - 1;
  }
}

// chlo.top_k(x, k) -> the first k entries of a stable descending sort of (x, position) along the last dim: largest
// values first, equal values in ascending position (the tie rule the reference keeps, src/pjrt_plugin/ops/
// sort_fft_complex.cc:40-82); floats compare in total order.
void lowerTopKIn(Region& r, int& nextId) {
  for (size_t k = 0; k < r.ops.size(); ++k) {
    Op* op = r.ops[k].get();
    for (auto& sub : op->regions) lowerTopKIn(*sub, nextId);
    if (op->name != "chlo.top_k") continue;
    if (op->operands.size() != 1 || op->results.size() != 2) throw CompileError("chlo.top_k: expected one operand and two results");
    Value* x = op->operands[0];
    const TensorType xt = x->type;
    if (xt.rank() < 1) throw CompileError("chlo.top_k: the operand must have at least one dim");
    const int64_t kk = op->integer("k");
    const int last = xt.rank() - 1;
    if (kk < 0 || kk > xt.dims[(size_t)last]) throw CompileError("chlo.top_k: k is out of range");
    const DType it = op->results[1]->type.dt;
    Rewriter rw{r, nextId, op->line, {}};
    TensorType idxT = xt;
    idxT.dt = it;
    auto io = makeOp("iota", {}, &r, op->line);
    Attr dimA;
    dimA.kind = Attr::Int;
    dimA.i = last;
    io->attrs["dim"] = dimA;
    Value* pos = rw.emit(std::move(io), idxT);
    // sort with the comparator "lhs > rhs" on the values
    auto so = makeOp("sort", {x, pos}, &r, op->line);
    Attr lastA = dimA;
    so->attrs["dimension"] = lastA;
    auto region = std::make_unique<Region>();
    region->parent = so.get();
    TensorType scalarV, scalarI, pred;
    scalarV.dt = xt.dt; scalarI.dt = it; pred.dt = DType::Pred;
    const TensorType argTypes[4] = {scalarV, scalarV, scalarI, scalarI};
    for (int a = 0; a < 4; ++a) {
      auto v = std::make_unique<Value>();
      v->id = nextId++;
      v->type = argTypes[a];
      v->argOf = region.get();
      v->defIndex = a;
      v->name = "%topk_arg" + std::to_string(v->id);
      region->args.push_back(std::move(v));
    }
    auto cmp = makeOp("compare", {region->args[0].get(), region->args[1].get()}, region.get(), op->line);
    Attr dir;
    dir.kind = Attr::Str;
    dir.s = "GT";
    cmp->attrs["direction"] = dir;
    if (isFloat(xt.dt)) {
      Attr ct;
      ct.kind = Attr::Str;
      ct.s = "TOTALORDER";
      cmp->attrs["compare_type"] = ct;
    }
    Value* gt = addResult(cmp.get(), pred, nextId);
    auto ret = makeOp("return", {gt}, region.get(), op->line);
    region->ops.push_back(std::move(cmp));
    region->ops.push_back(std::move(ret));
    so->regions.push_back(std::move(region));
    Value* sortedV = addResult(so.get(), xt, nextId);
    Value* sortedI = addResult(so.get(), idxT, nextId);
    rw.made.push_back(std::move(so));
    // first k along the last dim
    auto firstK = [&](Value* v) {
      auto sl = makeOp("slice", {v}, &r, op->line);
      std::vector<int64_t> start((size_t)xt.rank(), 0), limit = xt.dims, stride((size_t)xt.rank(), 1);
      limit[(size_t)last] = kk;
      sl->attrs["start"] = intsAttr(start);
      sl->attrs["limit"] = intsAttr(limit);
      sl->attrs["strides"] = intsAttr(stride);
      return sl;
    };
    auto sv = firstK(sortedV), si = firstK(sortedI);
    sv->results.push_back(std::move(op->results[0]));
    sv->results[0]->def = sv.get();
    si->results.push_back(std::move(op->results[1]));
    si->results[0]->def = si.get();
    rw.made.push_back(std::move(sv));
    rw.made.push_back(std::move(si));
    size_t nIns = rw.made.size();
    r.ops.erase(r.ops.begin() + k);
    r.ops.insert(r.ops.begin() + k, std::make_move_iterator(rw.made.begin()), std::make_move_iterator(rw.made.end()));
    k += nIns - 1;
  }
}

}  // namespace

// Ops of programs written for several devices that still reach a single-device plugin (reference:
// ops/collectives.cc:15-84 and ops/control_flow.cc:2266-2288).  With one device an all_reduce returns its operands,
// the partition and replica ids are zero, and a token, which only orders side effects that run in program order here
// anyway, is a float32 scalar placeholder (zero), also where it crosses the function boundary.  Anything that names
// more than one device is a compile error: treating it as the identity would silently give wrong values.
namespace {

void retypeTokens(Region& r) {
  for (auto& a : r.args) if (a->type.dt == DType::Token) { a->type.dt = DType::F32; a->type.dims.clear(); }
  for (auto& o : r.ops) {
    for (auto& v : o->results) if (v->type.dt == DType::Token) { v->type.dt = DType::F32; v->type.dims.clear(); }
    for (auto& sub : o->regions) retypeTokens(*sub);
  }
}

void lowerSingleDeviceOpsIn(Module& m, Region& r, int& nextId, VMap& repl) {
  for (size_t k = 0; k < r.ops.size(); ++k) {
    Op* op = r.ops[k].get();
    for (auto& sub : op->regions) lowerSingleDeviceOpsIn(m, *sub, nextId, repl);
    if (op->name == "all_reduce") {
      if (op->has("replica_groups")) {
        // members per group: the last dimension of a rank-2 tensor, else the element count (a flat list is one group)
        const Attr& a = op->attrs.at("replica_groups");
        int64_t perGroup = 0;
        if (a.dense) perGroup = a.dense->type.rank() >= 2 ? a.dense->type.dims.back() : a.dense->type.numel();
        else if (a.kind == Attr::Ints) perGroup = (int64_t)a.ints.size();
        else throw CompileError("stablehlo.all_reduce: replica_groups is not a tensor of integers");
        if (perGroup > 1) throw CompileError("stablehlo.all_reduce: multi-device all_reduce is not supported");
      }
      if (op->operands.size() != op->results.size()) throw CompileError("stablehlo.all_reduce: operand/result count mismatch");
      for (size_t i = 0; i < op->results.size(); ++i) repl[op->results[i].get()] = op->operands[i];
      r.ops.erase(r.ops.begin() + k);
      --k;
      continue;
    }
    const bool id = op->name == "partition_id" || op->name == "replica_id";
    const bool token = op->name == "create_token" || op->name == "after_all";
    if (!id && !token) continue;
    if (op->name == "partition_id" && m.numPartitions != 1) throw CompileError("stablehlo.partition_id: multi-partition execution is not supported");
    if (op->name == "replica_id" && m.numReplicas != 1) throw CompileError("stablehlo.replica_id: multi-replica execution is not supported");
    if (op->results.size() != 1) throw CompileError("stablehlo." + op->name + ": expected one result");
    TensorType t = op->results[0]->type;
    if (token) { t.dt = DType::F32; t.dims.clear(); }
    if (id && (t.rank() != 0 || !isInt(t.dt))) throw CompileError("stablehlo." + op->name + ": result must be a scalar integer tensor");
    Rewriter rw{r, nextId, op->line, {}};
    const uint64_t zero = 0;   // all-zero bytes are 0 of every integer type and 0.0f
    Value* c = rw.splat(t.dt, {}, &zero);
    repl[op->results[0].get()] = c;
    size_t nIns = rw.made.size();
    r.ops.erase(r.ops.begin() + k);
    r.ops.insert(r.ops.begin() + k, std::make_move_iterator(rw.made.begin()), std::make_move_iterator(rw.made.end()));
    k += nIns - 1;
  }
}

}  // namespace

// compare(v, 0, GT) next to maximum(v, 0) asks the same of the maximum: maximum(v, 0) > 0 exactly when v > 0 (a NaN
// stays a NaN and compares false either way).  The backward pass of a ReLU reads its mask this way; with the mask
// taken from the activation, the value before it has one reader left and the kernel that produces it can apply the
// maximum while it stores (planner.cc: the ReLU epilogue of small fp32 products).
namespace {
bool isZeroSplat(Value* v) {
  Op* d = v->def;
  while (d && (d->name == "broadcast_in_dim" || d->name == "reshape") && d->operands.size() == 1) d = d->operands[0]->def;
  if (!d || d->name != "constant" || !d->has("value") || !d->attrs.at("value").dense) return false;
  const DenseData& dd = *d->attrs.at("value").dense;
  if (!dd.splat && dd.type.numel() != 1) return false;
  if (dd.type.dt != DType::F32 || dd.bytes.size() < 4) return false;
  uint32_t bits;
  memcpy(&bits, dd.bytes.data(), 4);
  return (bits & 0x7FFFFFFFu) == 0;
}
// the other operand of maximum(v, 0) / maximum(0, v), or null
Value* reluInput(Op* op) {
  if (op->name != "maximum" || op->operands.size() != 2 || op->results.size() != 1) return nullptr;
  if (isZeroSplat(op->operands[1])) return op->operands[0];
  if (isZeroSplat(op->operands[0])) return op->operands[1];
  return nullptr;
}
void reluMasksIn(Region& r) {
  std::unordered_map<Value*, Value*> activationOf;   // v -> maximum(v, 0) seen earlier in this region
  for (auto& o : r.ops) {
    for (auto& sub : o->regions) reluMasksIn(*sub);
    if (Value* v = reluInput(o.get())) {
      if (v->type.dt == DType::F32) activationOf.emplace(v, o->result());
      continue;
    }
    if (o->name != "compare" || o->operands.size() != 2 || o->str("direction") != "GT") continue;
    auto it = activationOf.find(o->operands[0]);
    if (it == activationOf.end() || !isZeroSplat(o->operands[1])) continue;
    Value* v = o->operands[0];
    v->users.erase(std::remove(v->users.begin(), v->users.end(), o.get()), v->users.end());
    o->operands[0] = it->second;
    it->second->users.push_back(o.get());
  }
}
}  // namespace

void reluMasksFromActivations(Module& m) {
  for (auto& f : m.funcs) reluMasksIn(f->body);
}

void lowerSingleDeviceOps(Module& m) {
  Func* f = m.main();
  if (!f) return;
  int nextId = maxValueId(f->body) + 1;
  VMap repl;
  lowerSingleDeviceOpsIn(m, f->body, nextId, repl);
  if (!repl.empty()) applyReplacements(f->body, repl);
  retypeTokens(f->body);
  for (auto& t : f->resultTypes) if (t.dt == DType::Token) { t.dt = DType::F32; t.dims.clear(); }
}

// A reduction over no elements returns its init values: each result becomes a broadcast of the matching init operand.
namespace {
void lowerEmptyReductionsIn(Region& r) {
  for (size_t k = 0; k < r.ops.size(); ++k) {
    Op* op = r.ops[k].get();
    for (auto& sub : op->regions) lowerEmptyReductionsIn(*sub);
    if (op->name != "reduce" || op->operands.size() < 2 || op->operands.size() != 2 * op->results.size()) continue;
    if (op->operands[0]->type.numel() != 0 || op->results[0]->type.numel() == 0) continue;
    const size_t n = op->results.size();
    std::vector<std::unique_ptr<Op>> made;
    for (size_t j = 0; j < n; ++j) {
      auto bc = makeOp("broadcast_in_dim", {op->operands[n + j]}, &r, op->line);
      bc->attrs["dims"] = intsAttr({});
      bc->results.push_back(std::move(op->results[j]));
      bc->results[0]->def = bc.get();
      bc->results[0]->defIndex = 0;
      made.push_back(std::move(bc));
    }
    for (auto* o : op->operands) o->users.erase(std::remove(o->users.begin(), o->users.end(), op), o->users.end());
    for (auto& b : made) b->operands[0]->users.push_back(b.get());
    r.ops.erase(r.ops.begin() + (long)k);
    r.ops.insert(r.ops.begin() + (long)k, std::make_move_iterator(made.begin()), std::make_move_iterator(made.end()));
    k += n - 1;
  }
}
}  // namespace

void lowerEmptyReductions(Module& m) {
  if (Func* f = m.main()) lowerEmptyReductionsIn(f->body);
}

// A product step reads each operand as one strided matrix per batch: its free dims, its contracted dims and its batch
// dims each have to collapse to one stride (two for the batch).  jax leaves the operand dims of an einsum or tensordot
// where they are (free dims on both sides of a contracted one, say); such an operand gets a transpose in front, to
// [batch..., free..., contracted...] on the left and [batch..., contracted..., free...] on the right, which the result
// dims (batch, left free, right free) do not notice.  Reference: ops/linalg.cc:89-250 takes any dimension numbers.
namespace {
bool runCollapses(const TensorType& t, const std::vector<int64_t>& dims) {
  std::vector<int64_t> st((size_t)t.rank(), 1);
  for (int d = t.rank() - 2; d >= 0; --d) st[(size_t)d] = st[(size_t)d + 1] * t.dims[(size_t)d + 1];
  bool have = false;
  int64_t expect = 0;
  for (int64_t d : dims) {
    if (t.dims[(size_t)d] == 1) continue;
    if (have && st[(size_t)d] * t.dims[(size_t)d] != expect) return false;
    have = true;
    expect = st[(size_t)d];
  }
  return true;
}
void canonicalizeDotLayoutsIn(Region& r, int& nextId) {
  for (size_t k = 0; k < r.ops.size(); ++k) {
    Op* op = r.ops[k].get();
    for (auto& sub : op->regions) canonicalizeDotLayoutsIn(*sub, nextId);
    if (op->name != "dot_general" || op->operands.size() != 2) continue;
    Value* a = op->operands[0];
    Value* b = op->operands[1];
    if (!isFloat(a->type.dt)) continue;
    std::vector<int64_t> ab = op->ints("lhs_batch"), bb = op->ints("rhs_batch"), ac = op->ints("lhs_contract"), bc = op->ints("rhs_contract");
    auto has = [](const std::vector<int64_t>& v, int64_t x) { return std::find(v.begin(), v.end(), x) != v.end(); };
    std::vector<int64_t> af, bf;
    for (int d = 0; d < a->type.rank(); ++d) if (!has(ab, d) && !has(ac, d)) af.push_back(d);
    for (int d = 0; d < b->type.rank(); ++d) if (!has(bb, d) && !has(bc, d)) bf.push_back(d);
    // the contracted dims in the order of the left operand's memory, as the planner takes them
    std::vector<size_t> order(ac.size());
    for (size_t q = 0; q < order.size(); ++q) order[q] = q;
    std::sort(order.begin(), order.end(), [&](size_t x, size_t y) { return ac[x] < ac[y]; });
    std::vector<int64_t> acs, bcs;
    for (auto q : order) { acs.push_back(ac[q]); bcs.push_back(bc[q]); }
    // batch dims: at most two runs that collapse on both sides together
    size_t runs = 0;
    {
      std::vector<int64_t> sa((size_t)a->type.rank(), 1), sb((size_t)b->type.rank(), 1);
      for (int d = a->type.rank() - 2; d >= 0; --d) sa[(size_t)d] = sa[(size_t)d + 1] * a->type.dims[(size_t)d + 1];
      for (int d = b->type.rank() - 2; d >= 0; --d) sb[(size_t)d] = sb[(size_t)d + 1] * b->type.dims[(size_t)d + 1];
      int64_t ea = 0, eb = 0;
      for (size_t q = 0; q < ab.size(); ++q) {
        const int64_t n = a->type.dims[(size_t)ab[q]];
        if (n == 1) continue;
        if (runs == 0 || sa[(size_t)ab[q]] * n != ea || sb[(size_t)bb[q]] * n != eb) ++runs;
        ea = sa[(size_t)ab[q]];
        eb = sb[(size_t)bb[q]];
      }
    }
    const bool fine = runCollapses(a->type, acs) && runCollapses(b->type, bcs) && runCollapses(a->type, af) && runCollapses(b->type, bf) && runs <= 2;
    if (fine) continue;
    std::vector<std::unique_ptr<Op>> made;
    auto transposed = [&](Value* v, const std::vector<int64_t>& perm) -> Value* {
      bool identity = true;
      for (size_t q = 0; q < perm.size(); ++q) if (perm[q] != (int64_t)q) identity = false;
      if (identity) return v;
      auto t = makeOp("transpose", {v}, &r, op->line);
      t->attrs["dims"] = intsAttr(perm);
      TensorType tt = v->type;
      for (size_t q = 0; q < perm.size(); ++q) tt.dims[q] = v->type.dims[(size_t)perm[q]];
      Value* out = addResult(t.get(), tt, nextId);
      v->users.push_back(t.get());
      made.push_back(std::move(t));
      return out;
    };
    std::vector<int64_t> pa = ab, pb = bb;
    pa.insert(pa.end(), af.begin(), af.end());
    pa.insert(pa.end(), ac.begin(), ac.end());
    pb.insert(pb.end(), bc.begin(), bc.end());
    pb.insert(pb.end(), bf.begin(), bf.end());
    Value* na = transposed(a, pa);
    Value* nb = transposed(b, pb);
    auto swapOperand = [&](size_t at, Value* from, Value* to) {
      if (from == to) return;
      from->users.erase(std::remove(from->users.begin(), from->users.end(), op), from->users.end());
      op->operands[at] = to;
      to->users.push_back(op);
    };
    swapOperand(0, a, na);
    swapOperand(1, b, nb);
    const int64_t nbat = (int64_t)ab.size(), nfa = (int64_t)af.size(), nc = (int64_t)ac.size();
    std::vector<int64_t> batch, lc, rc;
    for (int64_t q = 0; q < nbat; ++q) batch.push_back(q);
    for (int64_t q = 0; q < nc; ++q) { lc.push_back(nbat + nfa + q); rc.push_back(nbat + q); }
    op->attrs["lhs_batch"] = intsAttr(batch);
    op->attrs["rhs_batch"] = intsAttr(batch);
    op->attrs["lhs_contract"] = intsAttr(lc);
    op->attrs["rhs_contract"] = intsAttr(rc);
    const size_t n = made.size();
    r.ops.insert(r.ops.begin() + (long)k, std::make_move_iterator(made.begin()), std::make_move_iterator(made.end()));
    k += n;
  }
}
}  // namespace

// float16 products and convolutions run on the float32 path: operands widened, the float32 result narrowed once
// (every f16 value is an f32 value, and the sums are accumulated in float32 as the fused kernels do for bf16).
namespace {
void widenHalfProductsIn(Region& r, int& nextId) {
  for (size_t k = 0; k < r.ops.size(); ++k) {
    Op* op = r.ops[k].get();
    for (auto& sub : op->regions) widenHalfProductsIn(*sub, nextId);
    if (op->name != "dot_general" && op->name != "dot" && op->name != "convolution") continue;
    if (op->operands.size() != 2 || op->results.size() != 1) continue;
    if (op->operands[0]->type.dt != DType::F16 && op->operands[1]->type.dt != DType::F16) continue;
    std::vector<std::unique_ptr<Op>> before;
    for (size_t q = 0; q < 2; ++q) {
      Value* v = op->operands[q];
      if (v->type.dt != DType::F16) continue;
      auto cv = makeOp("convert", {v}, &r, op->line);
      TensorType t = v->type;
      t.dt = DType::F32;
      Value* wide = addResult(cv.get(), t, nextId);
      v->users.erase(std::remove(v->users.begin(), v->users.end(), op), v->users.end());
      v->users.push_back(cv.get());
      op->operands[q] = wide;
      wide->users.push_back(op);
      before.push_back(std::move(cv));
    }
    Value* out = op->result();
    std::unique_ptr<Op> after;
    if (out->type.dt == DType::F16) {
      // the product keeps a new float32 result; the old result value (and its readers) moves to the narrowing convert
      after = makeOp("convert", {}, &r, op->line);
      after->results.push_back(std::move(op->results[0]));
      after->results[0]->def = after.get();
      after->results[0]->defIndex = 0;
      op->results.clear();
      TensorType t = after->results[0]->type;
      t.dt = DType::F32;
      Value* wide = addResult(op, t, nextId);
      after->operands.push_back(wide);
      wide->users.push_back(after.get());
    }
    const size_t nb = before.size();
    r.ops.insert(r.ops.begin() + (long)k, std::make_move_iterator(before.begin()), std::make_move_iterator(before.end()));
    k += nb;
    if (after) { r.ops.insert(r.ops.begin() + (long)k + 1, std::move(after)); ++k; }
  }
}
}  // namespace

// bitcast_convert between element types of different width (jnp's x.view(dtype), lax.bitcast_convert_type): to a narrower
// type the result gains a last dim of (wide / narrow) elements, least significant first; from a narrower type the last
// dim is folded into one element.  Written with same-width bitcasts, shifts by multiples of the narrow width and, for
// the widening form, an OR of the shifted parts.
namespace {
DType unsignedOfSize(size_t n) { return n == 1 ? DType::U8 : n == 2 ? DType::U16 : n == 4 ? DType::U32 : DType::U64; }
void lowerBitcastWidthsIn(Region& r, int& nextId) {
  for (size_t k = 0; k < r.ops.size(); ++k) {
    Op* op = r.ops[k].get();
    for (auto& sub : op->regions) lowerBitcastWidthsIn(*sub, nextId);
    if (op->name != "bitcast_convert" || op->operands.size() != 1 || op->results.size() != 1) continue;
    Value* x = op->operands[0];
    const TensorType rt = op->result()->type;
    if (x->type.dt == DType::Pred || rt.dt == DType::Pred) continue;
    const size_t a = dtypeSize(x->type.dt), b = dtypeSize(rt.dt);
    if (a == b) continue;
    Rewriter rw{r, nextId, op->line, {}};
    auto same = [&](Value* v, DType dt) -> Value* {   // same-width bitcast (a no-op when the type is already that)
      if (v->type.dt == dt) return v;
      TensorType t = v->type;
      t.dt = dt;
      return rw.unary("bitcast_convert", v, t);
    };
    auto shiftAmounts = [&](const TensorType& like, int64_t bitsPerStep) {   // iota along the last dim times the step, in `like`'s type
      auto io = makeOp("iota", {}, &r, op->line);
      Attr dimA;
      dimA.kind = Attr::Int;
      dimA.i = like.rank() - 1;
      io->attrs["dim"] = dimA;
      Value* pos = rw.emit(std::move(io), like);
      uint64_t step = (uint64_t)bitsPerStep;
      return rw.binary("multiply", pos, rw.splat(like.dt, like.dims, &step), like);
    };
    if (a > b) {
      const int64_t q = (int64_t)(a / b);
      if (rt.rank() != x->type.rank() + 1 || rt.dims.back() != q) throw CompileError("stablehlo.bitcast_convert: the result of a narrowing bitcast must add a last dim of " + std::to_string(q));
      const DType U = unsignedOfSize(a), Ub = unsignedOfSize(b);
      Value* bits = same(x, U);
      TensorType wide = rt;
      wide.dt = U;
      auto bc = makeOp("broadcast_in_dim", {bits}, &r, op->line);
      std::vector<int64_t> dims;
      for (int d = 0; d < x->type.rank(); ++d) dims.push_back(d);
      bc->attrs["dims"] = intsAttr(dims);
      Value* spread = rw.emit(std::move(bc), wide);
      Value* parts = rw.binary("shift_right_logical", spread, shiftAmounts(wide, (int64_t)b * 8), wide);
      TensorType narrow = rt;
      narrow.dt = Ub;
      if (rt.dt == Ub) {
        rw.finish(k, op, makeOp("convert", {parts}, &r, op->line));
      } else {
        Value* low = rw.unary("convert", parts, narrow);
        rw.finish(k, op, makeOp("bitcast_convert", {low}, &r, op->line));
      }
    } else {
      const int64_t q = (int64_t)(b / a);
      if (x->type.rank() != rt.rank() + 1 || x->type.dims.back() != q) throw CompileError("stablehlo.bitcast_convert: the operand of a widening bitcast must have a last dim of " + std::to_string(q));
      const DType Ua = unsignedOfSize(a), U = unsignedOfSize(b);
      Value* bits = same(x, Ua);
      TensorType wide = x->type;
      wide.dt = U;
      Value* ext = rw.unary("convert", bits, wide);
      Value* placed = rw.binary("shift_left", ext, shiftAmounts(wide, (int64_t)a * 8), wide);
      TensorType ut = rt;
      ut.dt = U;
      Value* acc = nullptr;
      for (int64_t j = 0; j < q; ++j) {
        std::vector<int64_t> start((size_t)wide.rank(), 0), count = wide.dims, stride((size_t)wide.rank(), 1);
        start.back() = j;
        count.back() = 1;
        Value* part = rw.unary("reshape", rw.slice(placed, start, count, stride), ut);
        acc = acc ? rw.binary("or", acc, part, ut) : part;
      }
      if (rt.dt == U) {
        // (the results move to an op of their own: OR with zero keeps the value)
        uint64_t zero = 0;
        rw.finish(k, op, makeOp("or", {acc, rw.splat(U, ut.dims, &zero)}, &r, op->line));
      } else {
        rw.finish(k, op, makeOp("bitcast_convert", {acc}, &r, op->line));
      }
    }
  }
}
}  // namespace

void lowerBitcastWidths(Module& m) {
  Func* f = m.main();
  if (!f) return;
  int nextId = maxValueId(f->body) + 1;
  lowerBitcastWidthsIn(f->body, nextId);
}

// Scatters on element types the scatter kernels do not take (bool, 8- and 16-bit integers, float16) run on the 32-bit
// type that holds them: operand and updates widened, the combiner retyped, the result narrowed.  Sums and products of
// narrow integers wrap the same way after one narrowing as after every step, a boolean sum is an OR (any count above
// zero is true), minima, maxima and plain writes are order-preserving under sign or zero extension.  Index tensors of
// 8 or 16 bits are widened to int32.
namespace {
void retypeRegion(Region& rg, DType from, DType to) {
  for (auto& a : rg.args) if (a->type.dt == from) a->type.dt = to;
  for (auto& o : rg.ops) {
    for (auto& v : o->results) if (v->type.dt == from) v->type.dt = to;
    for (auto& sub : o->regions) retypeRegion(*sub, from, to);
  }
}
void widenScatterTypesIn(Region& r, int& nextId) {
  for (size_t k = 0; k < r.ops.size(); ++k) {
    Op* op = r.ops[k].get();
    for (auto& sub : op->regions) widenScatterTypesIn(*sub, nextId);
    if (op->name != "scatter" || op->operands.size() != 3 || op->results.size() != 1 || op->regions.size() != 1) continue;
    std::vector<std::unique_ptr<Op>> before;
    auto converted = [&](size_t at, DType to) {
      Value* v = op->operands[at];
      auto cv = makeOp("convert", {v}, &r, op->line);
      TensorType t = v->type;
      t.dt = to;
      Value* w = addResult(cv.get(), t, nextId);
      v->users.erase(std::remove(v->users.begin(), v->users.end(), op), v->users.end());
      v->users.push_back(cv.get());
      op->operands[at] = w;
      w->users.push_back(op);
      before.push_back(std::move(cv));
    };
    const DType it = op->operands[1]->type.dt;
    if (it == DType::S8 || it == DType::U8 || it == DType::S16 || it == DType::U16) converted(1, DType::S32);
    const DType et = op->operands[0]->type.dt;
    DType wide = et;
    if (et == DType::F16) wide = DType::F32;
    else if (et == DType::S8 || et == DType::S16) wide = DType::S32;
    else if (et == DType::U8 || et == DType::U16 || et == DType::Pred) wide = DType::U32;
    std::unique_ptr<Op> after;
    if (wide != et && op->operands[2]->type.dt == et) {
      converted(0, wide);
      converted(2, wide);
      retypeRegion(*op->regions[0], et, wide);
      after = makeOp("convert", {}, &r, op->line);
      after->results.push_back(std::move(op->results[0]));
      after->results[0]->def = after.get();
      after->results[0]->defIndex = 0;
      op->results.clear();
      TensorType t = after->results[0]->type;
      t.dt = wide;
      Value* w = addResult(op, t, nextId);
      after->operands.push_back(w);
      w->users.push_back(after.get());
    }
    // A plain write of 64-bit elements moves two 32-bit halves: the same update wins both (updates are applied in
    // order), so operand and updates are read as [..., 2] uint32 tensors with the pair as one more window dim.
    // (lowerBitcastWidths, which runs later, spells the bitcasts out.)  Sums, minima and maxima of 64-bit elements
    // do not split this way and stay refused.
    Region& body = *op->regions[0];
    const bool plainWrite = body.args.size() == 2 && body.ops.size() == 1 && body.ops[0]->name == "return" && body.ops[0]->operands.size() == 1 &&
                            body.ops[0]->operands[0] == body.args[1].get();
    if ((et == DType::S64 || et == DType::U64) && op->operands[2]->type.dt == et && plainWrite) {
      auto halves = [&](size_t at) {
        Value* v = op->operands[at];
        auto bc = makeOp("bitcast_convert", {v}, &r, op->line);
        TensorType t = v->type;
        t.dt = DType::U32;
        t.dims.push_back(2);
        Value* w = addResult(bc.get(), t, nextId);
        v->users.erase(std::remove(v->users.begin(), v->users.end(), op), v->users.end());
        v->users.push_back(bc.get());
        op->operands[at] = w;
        w->users.push_back(op);
        before.push_back(std::move(bc));
      };
      const int64_t updatesRank = op->operands[2]->type.rank();
      halves(0);
      halves(2);
      auto uwd = op->ints("update_window_dims");
      uwd.push_back(updatesRank);
      op->attrs["update_window_dims"] = intsAttr(uwd);
      retypeRegion(body, et, DType::U32);
      after = makeOp("bitcast_convert", {}, &r, op->line);
      after->results.push_back(std::move(op->results[0]));
      after->results[0]->def = after.get();
      after->results[0]->defIndex = 0;
      op->results.clear();
      TensorType t = after->results[0]->type;
      t.dt = DType::U32;
      t.dims.push_back(2);
      Value* w = addResult(op, t, nextId);
      after->operands.push_back(w);
      w->users.push_back(after.get());
    }
    const size_t nb = before.size();
    if (nb == 0 && !after) continue;
    r.ops.insert(r.ops.begin() + (long)k, std::make_move_iterator(before.begin()), std::make_move_iterator(before.end()));
    k += nb;
    if (after) { r.ops.insert(r.ops.begin() + (long)k + 1, std::move(after)); ++k; }
  }
}
}  // namespace

void widenScatterTypes(Module& m) {
  Func* f = m.main();
  if (!f) return;
  int nextId = maxValueId(f->body) + 1;
  widenScatterTypesIn(f->body, nextId);
}

void widenHalfProducts(Module& m) {
  Func* f = m.main();
  if (!f) return;
  int nextId = maxValueId(f->body) + 1;
  widenHalfProductsIn(f->body, nextId);
}

void canonicalizeDotLayouts(Module& m) {
  Func* f = m.main();
  if (!f) return;
  int nextId = maxValueId(f->body) + 1;
  canonicalizeDotLayoutsIn(f->body, nextId);
}

void lowerTopK(Module& m) {
  Func* f = m.main();
  if (!f) return;
  int nextId = maxValueId(f->body) + 1;
  lowerTopKIn(f->body, nextId);
}

void lowerRng(Module& m) {
  Func* f = m.main();
  if (!f) return;
  int nextId = maxValueId(f->body) + 1;
  lowerRngIn(f->body, nextId);
}

void lowerWindowOps(Module& m) {
  Func* f = m.main();
  if (!f) return;
  int nextId = maxValueId(f->body) + 1;
  lowerWindowOpsIn(f->body, nextId);
}

void lowerGeneralScatters(Module& m) {
  Func* f = m.main();
  if (!f) return;
  int nextId = maxValueId(f->body) + 1;
  lowerScattersIn(f->body, nextId);
}

void eliminateDeadCode(Region& r) {
  std::unordered_map<const Value*, int> uses;
  collectUses(r, uses);
  while (sweep(r, uses)) {}
  removeDead(r);
}

void rebuildUses(Region& r) {
  std::function<void(Region&)> clear = [&](Region& q) {
    for (auto& a : q.args) a->users.clear();
    for (auto& o : q.ops) {
      for (auto& v : o->results) v->users.clear();
      for (auto& sub : o->regions) clear(*sub);
    }
  };
  std::function<void(Region&)> fill = [&](Region& q) {
    for (auto& o : q.ops) {
      for (auto* v : o->operands) v->users.push_back(o.get());
      for (auto& sub : o->regions) fill(*sub);
    }
  };
  clear(r);
  fill(r);
}

int countOps(const Region& r) {
  int n = 0;
  for (auto& o : r.ops) {
    ++n;
    for (auto& sub : o->regions) n += countOps(*sub);
  }
  return n;
}

static const std::set<std::string>& supportedOps() {
  static const std::set<std::string> s = {
      // elementwise (reference: ops/arithmetic.cc:535-607)
      "add", "subtract", "multiply", "divide", "maximum", "minimum", "power", "remainder", "atan2", "and", "or", "xor",
      "not", "negate", "abs", "exponential", "exponential_minus_one", "log", "log_plus_one", "sqrt", "rsqrt", "cbrt",
      "tanh", "tan", "sine", "cosine", "logistic", "floor", "ceil", "sign", "round_nearest_even", "round_nearest_afz",
      "is_finite", "shift_left", "shift_right_logical", "shift_right_arithmetic", "popcnt", "count_leading_zeros",
      "compare", "select", "clamp", "convert", "bitcast_convert", "reduce_precision",
      // shape / slicing (ops/shape.cc:260-270, ops/slice.cc:280-285)
      "constant", "iota", "reshape", "broadcast_in_dim", "transpose", "reverse", "concatenate", "slice", "dynamic_slice",
      "dynamic_update_slice", "pad",
      // heavy ops
      "reduce", "dot_general", "dot", "convolution", "gather", "scatter", "reduce_window", "select_and_scatter", "sort",
      // control flow (ops/control_flow.cc:2364-2376)
      "while", "case", "return", "optimization_barrier", "custom_call",
      // chlo unary ops (reference: ops/control_flow.cc:53-63)
      "chlo.asin", "chlo.acos", "chlo.atan", "chlo.sinh", "chlo.cosh", "chlo.asinh", "chlo.acosh", "chlo.atanh", "chlo.erf",
      "chlo.erf_inv",
  };
  return s;
}

// Attributes without which an op has no meaning.  The accessors of Op return 0 / an empty list for a missing key,
// which is right only where StableHLO defines that default, so the others are checked here once.
static void checkRequiredAttrs(const Op& o) {
  static const std::map<std::string, std::vector<const char*>> required = {
      {"iota", {"dim"}}, {"concatenate", {"dim"}}, {"broadcast_in_dim", {"dims"}}, {"transpose", {"dims"}},
      {"reverse", {"dims"}}, {"reduce", {"dimensions"}}, {"slice", {"start", "limit"}}, {"dynamic_slice", {"sizes"}},
      {"pad", {"low", "high"}}, {"compare", {"direction"}}, {"reduce_precision", {"exponent_bits", "mantissa_bits"}},
      {"constant", {"value"}}, {"gather", {"slice_sizes", "index_vector_dim", "start_index_map"}},
      {"scatter", {"index_vector_dim", "scatter_dims_to_operand_dims"}}, {"chlo.top_k", {"k"}},
      {"dot_general", {"lhs_contract", "rhs_contract"}}, {"custom_call", {"target"}}};
  auto it = required.find(o.name);
  if (it == required.end()) return;
  for (const char* k : it->second)
    if (!o.has(k))
      throw CompileError("stablehlo." + o.name + " at line " + std::to_string(o.line) + " lacks its '" + k + "' attribute");
  if (o.name == "reduce_precision" && (o.integer("exponent_bits") < 1 || o.integer("mantissa_bits") < 0))
    throw CompileError("stablehlo.reduce_precision at line " + std::to_string(o.line) + ": exponent_bits must be at least 1 and mantissa_bits non-negative");
}

static void scan(const Region& r, std::set<std::string>& bad) {
  for (auto& o : r.ops) {
    if (!supportedOps().count(o->name)) bad.insert(o->name);
    checkRequiredAttrs(*o);
    if (o->name == "custom_call") {
      const std::string& t = o->str("target");
      if (t != "Sharding" && t != "SPMDFullToShardShape" && t != "SPMDShardToFullShape") bad.insert("custom_call @" + t);
    }
    for (auto& sub : o->regions) scan(*sub, bad);
  }
}

void checkSupported(const Module& m) {
  std::set<std::string> bad;
  scan(m.main()->body, bad);
  if (bad.empty()) return;
  std::string msg = "unsupported StableHLO operation(s):";
  for (auto& b : bad) msg += " " + b;
  throw CompileError(msg);
}

}  // namespace mi355
