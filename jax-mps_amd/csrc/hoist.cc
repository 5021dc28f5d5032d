// Loop analysis and loop-invariant hoisting of products.
//
// A scan over a sequence (jax.lax.scan lowers to stablehlo.while, reference: ops/control_flow.cc:702-989) multiplies
// the step's input x[i] by a weight matrix in every iteration, and its backward loop recomputes the same products from
// saved values.  None of these depends on what the loop carries, so all iterations' products are one large product
// x[all] . W ahead of the loop; the body then reads slice i of the result.  What stays in the loop is the chain that
// really is sequential (the product with the carried state), and a step of the loop is one launch shorter.
#include <algorithm>
#include <cstdlib>
#include <functional>
#include <unordered_set>

#include "ir.h"

namespace mi355 {

bool constantInt(Value* v, int64_t& out) {
  Op* d = v->def;
  while (d && (d->name == "reshape" || d->name == "convert" || d->name == "broadcast_in_dim") && d->operands[0]->type.numel() == 1) d = d->operands[0]->def;
  if (!d || d->name != "constant") return false;
  auto& dd = *d->attrs.at("value").dense;
  if (!isInt(dd.type.dt) || dd.type.numel() != 1) return false;
  int64_t x = 0;
  size_t sz = dtypeSize(dd.type.dt);
  memcpy(&x, dd.bytes.data(), sz);
  if (isSignedInt(dd.type.dt) && sz < 8 && ((x >> (8 * sz - 1)) & 1)) x |= ~((int64_t(1) << (8 * sz)) - 1);
  out = x;
  return true;
}

int64_t staticTripCount(Op* op, LoopCounter* counter) {
  if (op->regions.size() != 2) return -1;
  Region& cond = *op->regions[0];
  Region& body = *op->regions[1];
  Op* ret = cond.terminator();
  if (!ret || ret->operands.size() != 1) return -1;
  Op* cmp = ret->operands[0]->def;
  if (!cmp || cmp->name != "compare") return -1;
  Value* lhs = cmp->operands[0];
  Value* rhs = cmp->operands[1];
  std::string dir = cmp->str("direction");
  int64_t limit;
  if (!(lhs->argOf == &cond) || !constantInt(rhs, limit)) {
    if (rhs->argOf == &cond && constantInt(lhs, limit)) {
      std::swap(lhs, rhs);
      dir = dir == "LT" ? "GT" : dir == "GT" ? "LT" : dir == "LE" ? "GE" : dir == "GE" ? "LE" : dir;
    } else {
      return -1;
    }
  }
  int ci = lhs->defIndex;
  int64_t init;
  if (!constantInt(op->operands[ci], init)) return -1;
  Value* next = body.terminator()->operands[ci];
  Op* add = next->def;
  if (!add || (add->name != "add" && add->name != "subtract")) return -1;
  int64_t step;
  Value* barg = body.args[ci].get();
  if (add->operands[0] == barg && constantInt(add->operands[1], step)) {
    if (add->name == "subtract") step = -step;
  } else if (add->name == "add" && add->operands[1] == barg && constantInt(add->operands[0], step)) {
  } else {
    return -1;
  }
  if (step == 0) return -1;
  int64_t n = 0;
  if (dir == "LT" && step > 0) n = limit > init ? (limit - init + step - 1) / step : 0;
  else if (dir == "LE" && step > 0) n = limit >= init ? (limit - init) / step + 1 : 0;
  else if (dir == "GT" && step < 0) n = init > limit ? (init - limit + (-step) - 1) / (-step) : 0;
  else if (dir == "GE" && step < 0) n = init >= limit ? (init - limit) / (-step) + 1 : 0;
  else if (dir == "NE" && (limit - init) % step == 0 && (limit - init) / step >= 0) n = (limit - init) / step;
  else return -1;
  if (counter) { counter->carry = ci; counter->init = init; counter->step = step; }
  return n;
}

namespace {

int maxId(const Region& r) {
  int m = -1;
  for (auto& a : r.args) m = std::max(m, a->id);
  for (auto& o : r.ops) {
    for (auto& v : o->results) m = std::max(m, v->id);
    for (auto& sub : o->regions) m = std::max(m, maxId(*sub));
  }
  return m;
}

// is `v` defined inside `body` (its arguments and nested regions included)?
bool definedIn(const Value* v, const Region* body) {
  const Region* r = v->def ? v->def->parent : v->argOf;
  while (r) {
    if (r == body) return true;
    r = r->parent ? r->parent->parent : nullptr;
  }
  return false;
}

struct WholeProduct {
  Region* region;
  Value *whole, *other;
  int side;
  std::vector<int64_t> contract, otherContract;
  Value* result;
};

struct Hoister {
  Op* loop;
  Region& body;
  int& nextId;
  std::vector<WholeProduct>& made_;   // whole products made so far, per region they were placed in

  // the value outside the loop that `v` stands for in every iteration, or null: something defined outside the body,
  // or a carry that the body hands on unchanged
  Value* invariant(Value* v) const {
    if (!definedIn(v, &body)) return v;
    if (v->argOf == &body) {
      Op* ret = body.terminator();
      const size_t k = (size_t)v->defIndex;
      if (ret && k < ret->operands.size() && ret->operands[k] == v && k < loop->operands.size()) return loop->operands[k];
    }
    return nullptr;
  }

  // a scalar integer that only the loop's scalar integer carries and constants determine
  bool pureIndex(Value* v, int depth = 0) const {
    if (depth > 16 || v->type.numel() != 1 || !(isInt(v->type.dt) || v->type.dt == DType::Pred)) return false;
    if (!definedIn(v, &body)) return true;
    if (v->argOf == &body) return true;
    Op* d = v->def;
    if (!d || d->parent != &body || d->results.size() != 1) return false;
    static const std::unordered_set<std::string> ok = {"constant", "add", "subtract", "multiply", "negate", "minimum", "maximum", "clamp", "select",
                                                       "compare", "convert", "reshape", "broadcast_in_dim", "remainder"};
    if (!ok.count(d->name)) return false;
    for (auto* o : d->operands) if (!pureIndex(o, depth + 1)) return false;
    return true;
  }

  struct Sliced {
    Value* whole = nullptr;   // the loop-invariant tensor, as named outside the loop
    int dim = -1;             // the dim the iteration selects one index of
    Value* index = nullptr;   // the start index along it (a value of the body)
  };

  // v = reshape(dynamic_slice(X, ..., i, ...)) that drops the one selected dim of a loop-invariant X
  bool slicedOperand(Value* v, Sliced& out) const {
    Op* rs = v->def;
    if (!rs || rs->parent != &body || rs->name != "reshape") return false;
    Op* ds = rs->operands[0]->def;
    if (!ds || ds->parent != &body || ds->name != "dynamic_slice") return false;
    Value* x = ds->operands[0];
    Value* whole = invariant(x);
    if (!whole) return false;
    const auto& sizes = ds->ints("sizes");
    const int rank = x->type.rank();
    if ((int)sizes.size() != rank || (int)ds->operands.size() != rank + 1) return false;
    int dim = -1;
    for (int d = 0; d < rank; ++d) {
      if (sizes[(size_t)d] == x->type.dims[(size_t)d]) continue;   // a full dim: the start is clamped to 0 whatever it is
      if (sizes[(size_t)d] != 1 || dim >= 0) return false;
      dim = d;
    }
    if (dim < 0 || !pureIndex(ds->operands[(size_t)dim + 1])) return false;
    std::vector<int64_t> dropped = x->type.dims;
    dropped.erase(dropped.begin() + dim);
    if (v->type.dims != dropped) return false;
    out.whole = whole;
    out.dim = dim;
    out.index = ds->operands[(size_t)dim + 1];
    return true;
  }

  Value* addResult(Op* op, const TensorType& t) {
    auto v = std::make_unique<Value>();
    v->id = nextId++;
    v->type = t;
    v->def = op;
    v->defIndex = (int)op->results.size();
    v->name = "%hoisted" + std::to_string(v->id);
    op->results.push_back(std::move(v));
    return op->results.back().get();
  }

  static Attr intsAttr(const std::vector<int64_t>& v) {
    Attr a;
    a.kind = Attr::Ints;
    a.ints = v;
    return a;
  }

  // returns the ops to place ahead of the loop; rewrites the body in place
  std::vector<std::unique_ptr<Op>> run(int64_t trip) {
    std::vector<std::unique_ptr<Op>> ahead;
    Region* outer = loop->parent;
    for (size_t k = 0; k < body.ops.size(); ++k) {
      Op* dot = body.ops[k].get();
      if (dot->name != "dot_general" || !dot->ints("lhs_batch").empty() || !dot->ints("rhs_batch").empty()) continue;
      Value* a = dot->operands[0];
      Value* b = dot->operands[1];
      Value* c = dot->result();
      if (a->type.dt != b->type.dt || (a->type.dt != DType::F32 && a->type.dt != DType::BF16) || c->type.numel() == 0) continue;
      Sliced sl;
      int side = -1;
      Value* other = nullptr;
      if (slicedOperand(a, sl) && (other = invariant(b))) side = 0;
      else if (slicedOperand(b, sl) && (other = invariant(a))) side = 1;
      if (side < 0) continue;
      const int64_t n = sl.whole->type.dims[(size_t)sl.dim];
      // worth it when the loop visits most of the slices, and the results of all iterations stay a modest buffer
      if (n < 2 || n > 2 * trip || (int64_t)c->type.bytes() * n > ((int64_t)256 << 20)) continue;
      // the product over the whole tensor: the selected dim is one more free dim of its side
      std::vector<int64_t> contract = dot->ints(side == 0 ? "lhs_contract" : "rhs_contract");
      for (auto& d : contract) if (d >= sl.dim) ++d;
      auto isContract = [&](int64_t d) { return std::find(contract.begin(), contract.end(), d) != contract.end(); };
      // the product kernels read an operand whose free dims are one run of neighbouring dims (they collapse to one
      // strided dim); a selected dim apart from the other free dims would ask for a transposed copy of the whole tensor
      {
        std::vector<int> freeDims;
        for (int d = 0; d < sl.whole->type.rank(); ++d) if (!isContract(d)) freeDims.push_back(d);
        if (freeDims.back() - freeDims.front() + 1 != (int)freeDims.size()) continue;
        if (!contract.empty()) {
          const auto mm = std::minmax_element(contract.begin(), contract.end());
          if (*mm.second - *mm.first + 1 != (int64_t)contract.size()) continue;   // the same for the contracted dims
        }
      }
      int before = 0;   // free dims of the sliced side ahead of the selected one
      for (int d = 0; d < sl.dim; ++d) if (!isContract(d)) ++before;
      const int lhsFree = a->type.rank() - (int)dot->ints("lhs_contract").size();
      const int pos = side == 0 ? before : lhsFree + before;
      TensorType wholeT = c->type;
      wholeT.dims.insert(wholeT.dims.begin() + pos, n);
      // (a backward loop recomputes the forward loop's products: the same whole product serves both)
      Value* all = nullptr;
      const std::vector<int64_t>& otherContract = dot->ints(side == 0 ? "rhs_contract" : "lhs_contract");
      for (auto& m : made_)
        if (m.region == outer && m.whole == sl.whole && m.other == other && m.side == side && m.contract == contract &&
            m.otherContract == otherContract && m.result->type == wholeT)
          all = m.result;
      if (!all) {
        auto big = std::make_unique<Op>();
        big->name = "dot_general";
        big->operands = side == 0 ? std::vector<Value*>{sl.whole, other} : std::vector<Value*>{other, sl.whole};
        big->attrs = dot->attrs;
        big->attrs[side == 0 ? "lhs_contract" : "rhs_contract"] = intsAttr(contract);
        big->parent = outer;
        big->line = dot->line;
        all = addResult(big.get(), wholeT);
        ahead.push_back(std::move(big));
        made_.push_back({outer, sl.whole, other, side, contract, otherContract, all});
      }
      // in the body: slice `pos` of the result at the same index, then drop the unit dim
      std::vector<std::unique_ptr<Op>> made;
      auto zero = std::make_unique<Op>();
      zero->name = "constant";
      zero->parent = &body;
      zero->line = dot->line;
      Attr dv;
      dv.kind = Attr::Dense;
      dv.dense = std::make_shared<DenseData>();
      dv.dense->type.dt = sl.index->type.dt;
      dv.dense->splat = true;
      dv.dense->bytes.assign(dtypeSize(sl.index->type.dt), 0);
      zero->attrs["value"] = dv;
      TensorType scalar;
      scalar.dt = sl.index->type.dt;
      Value* z = addResult(zero.get(), scalar);
      made.push_back(std::move(zero));
      Value* index = sl.index;
      if (index->type.rank() != 0) {
        auto flat = std::make_unique<Op>();
        flat->name = "reshape";
        flat->operands = {index};
        flat->parent = &body;
        flat->line = dot->line;
        index = addResult(flat.get(), scalar);
        made.push_back(std::move(flat));
      }
      auto ds = std::make_unique<Op>();
      ds->name = "dynamic_slice";
      ds->operands = {all};
      std::vector<int64_t> sizes = wholeT.dims;
      sizes[(size_t)pos] = 1;
      for (int d = 0; d < wholeT.rank(); ++d) ds->operands.push_back(d == pos ? index : z);
      ds->attrs["sizes"] = intsAttr(sizes);
      ds->parent = &body;
      ds->line = dot->line;
      TensorType sliceT = wholeT;
      sliceT.dims = sizes;
      Value* one = addResult(ds.get(), sliceT);
      made.push_back(std::move(ds));
      auto rs = std::make_unique<Op>();
      rs->name = "reshape";
      rs->operands = {one};
      rs->parent = &body;
      rs->line = dot->line;
      rs->results = std::move(dot->results);   // takes over the product's value: its readers need no rewiring
      for (auto& v : rs->results) v->def = rs.get();
      made.push_back(std::move(rs));
      const size_t added = made.size();
      body.ops.erase(body.ops.begin() + (long)k);
      body.ops.insert(body.ops.begin() + (long)k, std::make_move_iterator(made.begin()), std::make_move_iterator(made.end()));
      k += added - 1;
    }
    return ahead;
  }
};

void hoistIn(Region& r, int& nextId, std::vector<WholeProduct>& made) {
  for (size_t k = 0; k < r.ops.size(); ++k) {
    Op* op = r.ops[k].get();
    for (auto& sub : op->regions) hoistIn(*sub, nextId, made);
    if (op->name != "while" || op->regions.size() != 2) continue;
    const int64_t trip = staticTripCount(op);
    if (trip < 2) continue;
    Hoister h{op, *op->regions[1], nextId, made};
    auto ahead = h.run(trip);
    const size_t n = ahead.size();
    r.ops.insert(r.ops.begin() + (long)k, std::make_move_iterator(ahead.begin()), std::make_move_iterator(ahead.end()));
    k += n;
  }
}

}  // namespace

// ---- updates masked by their own index check ---------------------------------------------------------------
// JAX's x.at[i].add(u) zeroes the update rows whose index is out of range, select(in_range(i), u, 0), before a scatter
// that ignores exactly those rows anyway (out-of-range scatter indices are dropped by definition).  For a whole-row
// scatter along dim 0 whose indices are that same i, the select changes nothing the scatter reads: it takes u
// itself, and the pass over the updates that only rewrote them is gone.
namespace {

bool isRowMaskOfIndex(Value* mask, Value* index, int64_t rows, int updRank) {
  Op* bc = mask->def;
  if (!bc || bc->name != "broadcast_in_dim" || (int)mask->type.rank() != updRank) return false;
  Value* p = bc->operands[0];
  const auto& dims = bc->ints("dims");
  if (p->type.rank() != 1 || dims != std::vector<int64_t>{0} || p->type.dims[0] != index->type.dims[0]) return false;
  Op* both = p->def;
  if (!both || both->name != "and") return false;
  bool lower = false, upper = false;
  for (Value* side : both->operands) {
    Op* c = side->def;
    if (!c || c->name != "compare" || !isSignedInt(c->operands[0]->type.dt)) return false;
    const std::string& dir = c->str("direction");
    int64_t k;
    if (c->operands[0] == index && constantInt(c->operands[1], k)) {
      if (dir == "GE" && k <= 0) lower = true;                                   // holds for every index >= 0
      else if (dir == "GT" && k < 0) lower = true;
      else if ((dir == "LE" && k >= rows - 1) || (dir == "LT" && k >= rows)) upper = true;   // holds for every index < rows
      else return false;
    } else if (c->operands[1] == index && constantInt(c->operands[0], k)) {
      if (dir == "LE" && k <= 0) lower = true;
      else if (dir == "LT" && k < 0) lower = true;
      else if ((dir == "GE" && k >= rows - 1) || (dir == "GT" && k >= rows)) upper = true;
      else return false;
    } else {
      return false;
    }
  }
  return lower && upper;
}

void dropMasksIn(Region& r) {
  for (auto& op : r.ops) {
    for (auto& sub : op->regions) dropMasksIn(*sub);
    if (op->name != "scatter" || op->operands.size() != 3) continue;
    Value* operand = op->operands[0];
    Value* idx = op->operands[1];
    Value* upd = op->operands[2];
    if (operand->type.rank() < 1 || op->ints("inserted_window_dims") != std::vector<int64_t>{0} ||
        op->ints("scatter_dims_to_operand_dims") != std::vector<int64_t>{0} || !op->ints("input_batching_dims").empty())
      continue;
    // one scatter dim in front: updates [n, row...], indices [n] or [n, 1]
    if (upd->type.rank() != operand->type.rank() || idx->type.numel() != upd->type.dims[0]) continue;
    Value* index = idx;
    if (index->def && index->def->name == "reshape") index = index->def->operands[0];
    if (index->type.rank() != 1 || !isSignedInt(index->type.dt)) continue;
    Op* sel = upd->def;
    if (!sel || sel->name != "select" || sel->operands.size() != 3) continue;
    if (!isRowMaskOfIndex(sel->operands[0], index, operand->type.dims[0], upd->type.rank())) continue;
    if (!(sel->operands[1]->type == upd->type)) continue;
    op->operands[2] = sel->operands[1];
  }
}

}  // namespace

void dropScatterIndexMasks(Module& m) {
  if (getenv("MI355X_SCATTER_MASKS") && atoi(getenv("MI355X_SCATTER_MASKS")) != 0) return;   // 1 keeps the masks
  if (Func* f = m.main()) dropMasksIn(f->body);
}

void hoistLoopProducts(Module& m) {
  if (getenv("MI355X_HOIST_PRODUCTS") && atoi(getenv("MI355X_HOIST_PRODUCTS")) == 0) return;
  Func* f = m.main();
  if (!f) return;
  int nextId = maxId(f->body) + 1;
  std::vector<WholeProduct> made;
  hoistIn(f->body, nextId, made);
}

}  // namespace mi355
