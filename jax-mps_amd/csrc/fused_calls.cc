// The fused-op custom calls of the reference's Python layer, accepted at the PJRT boundary.
//
// The reference's jax_plugins.mps.ops registers JAX primitives whose lowering is a stablehlo.custom_call with a
// target name and a JSON backend_config (src/jax_plugins/mps/ops.py:52-596); its executor maps each target to an
// mlx::core::fast routine (src/pjrt_plugin/ops/control_flow.cc:1484-1533 sdpa / sdpa_causal, :1676-1697 rms_norm,
// :1749-1800 layer_norm and its backward, :1804-1831 rope, :1835-1858 gelu, :1863-2020 the backward forms).  Here
// each call is rewritten, before inlining, into a call of a private function written in plain StableHLO for the
// call's shapes; the planner then fuses that text like any other: the attention chain is what
// planner.cc::matchAttention turns into one launch of the bf16 attention kernel, the norms become row programs, rope
// and gelu elementwise kernels.  The definitions follow the reference's own fallback implementations
// (ops.py:63-76, 99-107, 258-262, 337-343, 418-438, 539-552), computing in float32 and rounding once to the operand
// type, as the fused routines they stand for do.  Both the reference's target names ("mps.<op>") and this plugin's
// own ("mi355x.<op>") are accepted.
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <functional>
#include <sstream>

#include "ir.h"

namespace mi355 {

namespace {

struct V {
  std::string name;
  TensorType t;
};

std::string ints(const std::vector<int64_t>& v) {
  std::string s;
  for (size_t k = 0; k < v.size(); ++k) s += (k ? ", " : "") + std::to_string(v[k]);
  return s;
}

std::string floatLit(double x) {
  if (std::isinf(x)) return x > 0 ? "0x7F800000" : "0xFF800000";
  char buf[64];
  snprintf(buf, sizeof buf, "%.9e", x);
  return buf;
}

// Writes the body of one function in the pretty StableHLO forms the front end reads.
struct Text {
  std::ostringstream os;
  int n = 0;
  std::vector<V> args;

  TensorType ty(DType dt, std::vector<int64_t> dims) {
    TensorType t;
    t.dt = dt;
    t.dims = std::move(dims);
    return t;
  }
  V fresh(const TensorType& t) { return V{"%v" + std::to_string(n++), t}; }
  V arg(const TensorType& t) {
    V v{"%arg" + std::to_string(args.size()), t};
    args.push_back(v);
    return v;
  }
  V scalar(double x, DType dt) {
    V v = fresh(ty(dt, {}));
    os << "    " << v.name << " = stablehlo.constant dense<" << (isFloat(dt) ? floatLit(x) : std::to_string((long long)x)) << "> : " << v.t.str() << "\n";
    return v;
  }
  V bcast(const V& x, const std::vector<int64_t>& shape, const std::vector<int64_t>& dims) {
    if (x.t.dims == shape) return x;
    V v = fresh(ty(x.t.dt, shape));
    os << "    " << v.name << " = stablehlo.broadcast_in_dim " << x.name << ", dims = [" << ints(dims) << "] : (" << x.t.str() << ") -> " << v.t.str() << "\n";
    return v;
  }
  V splat(double x, const TensorType& like) { return bcast(scalar(x, like.dt), like.dims, {}); }
  // trailing-aligned (numpy) broadcast of x to `shape`
  V bcastTo(const V& x, const std::vector<int64_t>& shape) {
    if (x.t.dims == shape) return x;
    const size_t off = shape.size() - x.t.dims.size();
    std::vector<int64_t> dims;
    for (size_t k = 0; k < x.t.dims.size(); ++k) dims.push_back((int64_t)(off + k));
    return bcast(x, shape, dims);
  }
  V binary(const char* op, V a, V b) {
    if (a.t.dims != b.t.dims) {
      if (a.t.numel() >= b.t.numel()) b = bcastTo(b, a.t.dims);
      else a = bcastTo(a, b.t.dims);
    }
    V v = fresh(a.t);
    os << "    " << v.name << " = stablehlo." << op << " " << a.name << ", " << b.name << " : " << v.t.str() << "\n";
    return v;
  }
  V add(const V& a, const V& b) { return binary("add", a, b); }
  V sub(const V& a, const V& b) { return binary("subtract", a, b); }
  V mul(const V& a, const V& b) { return binary("multiply", a, b); }
  V div(const V& a, const V& b) { return binary("divide", a, b); }
  V mulc(const V& a, double c) { return mul(a, splat(c, a.t)); }
  V addc(const V& a, double c) { return add(a, splat(c, a.t)); }
  V unary(const char* op, const V& x) {
    V v = fresh(x.t);
    os << "    " << v.name << " = stablehlo." << op << " " << x.name << " : " << v.t.str() << "\n";
    return v;
  }
  V convert(const V& x, DType dt) {
    if (x.t.dt == dt) return x;
    V v = fresh(ty(dt, x.t.dims));
    os << "    " << v.name << " = stablehlo.convert " << x.name << " : (" << x.t.str() << ") -> " << v.t.str() << "\n";
    return v;
  }
  V compare(const char* dir, const V& a, const V& b) {
    V v = fresh(ty(DType::Pred, a.t.dims));
    os << "    " << v.name << " = stablehlo.compare  " << dir << ", " << a.name << ", " << b.name << ",  " << (isFloat(a.t.dt) ? "FLOAT" : "SIGNED") << " : ("
       << a.t.str() << ", " << b.t.str() << ") -> " << v.t.str() << "\n";
    return v;
  }
  V select(const V& p, const V& a, const V& b) {
    V v = fresh(a.t);
    os << "    " << v.name << " = stablehlo.select " << p.name << ", " << a.name << ", " << b.name << " : " << p.t.str() << ", " << v.t.str() << "\n";
    return v;
  }
  V reshape(const V& x, const std::vector<int64_t>& shape) {
    if (x.t.dims == shape) return x;
    V v = fresh(ty(x.t.dt, shape));
    os << "    " << v.name << " = stablehlo.reshape " << x.name << " : (" << x.t.str() << ") -> " << v.t.str() << "\n";
    return v;
  }
  V iota(DType dt, const std::vector<int64_t>& shape, int dim) {
    V v = fresh(ty(dt, shape));
    os << "    " << v.name << " = stablehlo.iota dim = " << dim << " : " << v.t.str() << "\n";
    return v;
  }
  V slice(const V& x, int dim, int64_t start, int64_t limit, int64_t stride = 1) {
    std::vector<int64_t> shape = x.t.dims;
    shape[(size_t)dim] = (limit - start + stride - 1) / stride;
    V v = fresh(ty(x.t.dt, shape));
    os << "    " << v.name << " = stablehlo.slice " << x.name << " [";
    for (size_t k = 0; k < x.t.dims.size(); ++k) {
      if (k) os << ", ";
      if ((int)k == dim) { os << start << ":" << limit; if (stride != 1) os << ":" << stride; }
      else os << "0:" << x.t.dims[k];
    }
    os << "] : (" << x.t.str() << ") -> " << v.t.str() << "\n";
    return v;
  }
  V concat(const std::vector<V>& xs, int dim) {
    if (xs.size() == 1) return xs[0];
    std::vector<int64_t> shape = xs[0].t.dims;
    shape[(size_t)dim] = 0;
    for (auto& x : xs) shape[(size_t)dim] += x.t.dims[(size_t)dim];
    V v = fresh(ty(xs[0].t.dt, shape));
    os << "    " << v.name << " = stablehlo.concatenate ";
    for (size_t k = 0; k < xs.size(); ++k) os << (k ? ", " : "") << xs[k].name;
    os << ", dim = " << dim << " : (";
    for (size_t k = 0; k < xs.size(); ++k) os << (k ? ", " : "") << xs[k].t.str();
    os << ") -> " << v.t.str() << "\n";
    return v;
  }
  V reduce(const char* op, const V& x, const std::vector<int64_t>& dims, double init) {
    std::vector<int64_t> shape;
    for (size_t k = 0; k < x.t.dims.size(); ++k) {
      bool red = false;
      for (auto d : dims) red = red || (size_t)d == k;
      if (!red) shape.push_back(x.t.dims[k]);
    }
    V c = scalar(init, x.t.dt);
    V v = fresh(ty(x.t.dt, shape));
    os << "    " << v.name << " = stablehlo.reduce(" << x.name << " init: " << c.name << ") applies stablehlo." << op << " across dimensions = [" << ints(dims)
       << "] : (" << x.t.str() << ", " << c.t.str() << ") -> " << v.t.str() << "\n";
    return v;
  }
  // value reduced over `dims`, broadcast back to x's shape
  V reduceBack(const char* op, const V& x, const std::vector<int64_t>& dims, double init) {
    V r = reduce(op, x, dims, init);
    std::vector<int64_t> keep;
    for (size_t k = 0; k < x.t.dims.size(); ++k) {
      bool red = false;
      for (auto d : dims) red = red || (size_t)d == k;
      if (!red) keep.push_back((int64_t)k);
    }
    return bcast(r, x.t.dims, keep);
  }
  V rowMean(const V& x) {
    const int64_t last = (int64_t)x.t.dims.size() - 1;
    return mulc(reduceBack("add", x, {last}, 0.0), 1.0 / (double)x.t.dims.back());
  }
  V dot(const V& a, const V& b, const std::vector<int64_t>& ba, const std::vector<int64_t>& bb, const std::vector<int64_t>& ca,
        const std::vector<int64_t>& cb, DType out) {
    auto in = [](const std::vector<int64_t>& v, size_t k) { for (auto d : v) if ((size_t)d == k) return true; return false; };
    std::vector<int64_t> shape;
    for (auto d : ba) shape.push_back(a.t.dims[(size_t)d]);
    for (size_t k = 0; k < a.t.dims.size(); ++k) if (!in(ba, k) && !in(ca, k)) shape.push_back(a.t.dims[k]);
    for (size_t k = 0; k < b.t.dims.size(); ++k) if (!in(bb, k) && !in(cb, k)) shape.push_back(b.t.dims[k]);
    V v = fresh(ty(out, shape));
    os << "    " << v.name << " = stablehlo.dot_general " << a.name << ", " << b.name << ", ";
    if (!ba.empty()) os << "batching_dims = [" << ints(ba) << "] x [" << ints(bb) << "], ";
    os << "contracting_dims = [" << ints(ca) << "] x [" << ints(cb) << "], precision = [DEFAULT, DEFAULT] : (" << a.t.str() << ", " << b.t.str() << ") -> "
       << v.t.str() << "\n";
    return v;
  }

  std::string function(const std::string& name, const std::vector<V>& results) {
    std::ostringstream f;
    f << "module {\n  func.func private @" << name << "(";
    for (size_t k = 0; k < args.size(); ++k) f << (k ? ", " : "") << args[k].name << ": " << args[k].t.str();
    f << ") -> (";
    for (size_t k = 0; k < results.size(); ++k) f << (k ? ", " : "") << results[k].t.str();
    f << ") {\n" << os.str() << "    return ";
    for (size_t k = 0; k < results.size(); ++k) f << (k ? ", " : "") << results[k].name;
    f << " : ";
    for (size_t k = 0; k < results.size(); ++k) f << (k ? ", " : "") << results[k].t.str();
    f << "\n  }\n}\n";
    return f.str();
  }
};

// "key": value pairs of a backend_config such as {"scale": 0.125, "traditional": false}
struct Config {
  std::string text;
  bool find(const std::string& key, std::string& out) const {
    const std::string q = "\"" + key + "\"";
    size_t p = text.find(q);
    if (p == std::string::npos) return false;
    p = text.find(':', p + q.size());
    if (p == std::string::npos) return false;
    ++p;
    while (p < text.size() && (text[p] == ' ' || text[p] == '\t')) ++p;
    size_t e = p;
    while (e < text.size() && text[e] != ',' && text[e] != '}' && text[e] != ' ') ++e;
    out = text.substr(p, e - p);
    return !out.empty();
  }
  double number(const std::string& key, double dflt) const {
    std::string s;
    return find(key, s) ? atof(s.c_str()) : dflt;
  }
  bool boolean(const std::string& key, bool dflt) const {
    std::string s;
    if (!find(key, s)) return dflt;
    return s == "true" || s == "True" || s == "1";
  }
};

[[noreturn]] void bad(const std::string& target, const std::string& what) { throw CompileError("stablehlo.custom_call @" + target + ": " + what); }

const float kMostNegative = -3.40282347e38f;   // finfo(float32).min: what a masked score becomes (ops.py:72)

// ---- attention ------------------------------------------------------------------------------------------------------
struct Attention {
  V q, k, v;          // [B, N, T, H], [B, N, S, H] (key / value heads already repeated to N), [B, N, S, H]
  V p;                // softmax probabilities, float32 [B, N, T, S]
  int64_t B, N, Nkv, T, S, H;
};

// scores, mask and softmax shared by the forward and backward forms; `mask` may be null (causal builds its own)
Attention attentionProbabilities(Text& t, const std::string& target, const V& q, const V& k0, const V& v0, const V* mask, bool causal, double scale) {
  if (q.t.rank() != 4 || k0.t.rank() != 4 || v0.t.rank() != 4) bad(target, "queries, keys and values must have four dims (B, N, T, H)");
  Attention a;
  a.B = q.t.dims[0]; a.N = q.t.dims[1]; a.T = q.t.dims[2]; a.H = q.t.dims[3];
  a.Nkv = k0.t.dims[1]; a.S = k0.t.dims[2];
  if (k0.t.dims != v0.t.dims || k0.t.dims[0] != a.B || k0.t.dims[3] != a.H || a.Nkv <= 0 || a.N % a.Nkv != 0)
    bad(target, "keys and values must be (B, N_kv, S, H) with N a multiple of N_kv");
  if (q.t.dt != k0.t.dt || q.t.dt != v0.t.dt || !isFloat(q.t.dt)) bad(target, "queries, keys and values must share one float type");
  auto repeatHeads = [&](const V& x) {
    if (a.Nkv == a.N) return x;
    const int64_t g = a.N / a.Nkv;
    V r = t.reshape(x, {a.B, a.Nkv, 1, a.S, a.H});
    r = t.bcast(r, {a.B, a.Nkv, g, a.S, a.H}, {0, 1, 2, 3, 4});
    return t.reshape(r, {a.B, a.N, a.S, a.H});
  };
  a.q = q; a.k = repeatHeads(k0); a.v = repeatHeads(v0);
  V s = t.dot(a.q, a.k, {0, 1}, {0, 1}, {3}, {3}, DType::F32);
  s = t.mulc(s, scale);
  V gate;          // boolean [b, n, t, s] with ones where it broadcasts
  if (causal) {
    // query t sees keys up to t + (S - T): the last query sees every key (what the fused routine's "causal" mode does)
    V qi = t.addc(t.iota(DType::S32, {1, 1, a.T, a.S}, 2), (double)(a.S - a.T));
    V ki = t.iota(DType::S32, {1, 1, a.T, a.S}, 3);
    gate = t.compare("LE", ki, qi);
  } else if (mask) {
    if (mask->t.rank() > 4) bad(target, "the mask must broadcast to (B, N, T, S)");
    std::vector<int64_t> md(4 - (size_t)mask->t.rank(), 1);
    for (auto d : mask->t.dims) md.push_back(d);
    const int64_t full[4] = {a.B, a.N, a.T, a.S};
    for (int d = 0; d < 4; ++d) if (md[(size_t)d] != 1 && md[(size_t)d] != full[d]) bad(target, "the mask must broadcast to (B, N, T, S)");
    V m4 = t.reshape(*mask, md);
    if (mask->t.dt == DType::Pred) gate = m4;
    else if (isFloat(mask->t.dt)) s = t.add(s, t.bcast(t.convert(m4, DType::F32), s.t.dims, {0, 1, 2, 3}));   // additive bias (ops.py:69-70)
    else bad(target, "the mask must be boolean or floating");
  }
  if (!gate.name.empty()) s = t.select(t.bcast(gate, s.t.dims, {0, 1, 2, 3}), s, t.splat(kMostNegative, s.t));
  V centred = t.sub(s, t.reduceBack("maximum", s, {3}, -INFINITY));
  V e = t.unary("exponential", centred);
  a.p = t.div(e, t.reduceBack("add", e, {3}, 0.0));
  return a;
}

std::string sdpaForward(const std::string& target, const std::string& fn, const std::vector<TensorType>& in, bool causal, const Config& c) {
  Text t;
  V q = t.arg(in[0]), k = t.arg(in[1]), v = t.arg(in[2]);
  V mask;
  if (!causal) mask = t.arg(in[3]);
  Attention a = attentionProbabilities(t, target, q, k, v, causal ? nullptr : &mask, causal, c.number("scale", 1.0));
  V out = t.dot(t.convert(a.p, q.t.dt), a.v, {0, 1}, {0, 1}, {3}, {2}, q.t.dt);
  return t.function(fn, {out});
}

// dq, dk, dv with the probabilities recomputed (reference: vjp of the forward routine, control_flow.cc:1863-1924)
std::string sdpaBackward(const std::string& target, const std::string& fn, const std::vector<TensorType>& in, bool causal, const Config& c) {
  Text t;
  V q = t.arg(in[0]), k = t.arg(in[1]), v = t.arg(in[2]);
  V mask;
  if (!causal) mask = t.arg(in[3]);
  V g = t.arg(in[causal ? 3 : 4]);
  if (!(g.t == q.t)) bad(target, "the output gradient must have the queries' type");
  const double scale = c.number("scale", 1.0);
  Attention a = attentionProbabilities(t, target, q, k, v, causal ? nullptr : &mask, causal, scale);
  const DType dt = q.t.dt;
  const bool grouped = a.Nkv != a.N;
  V pd = t.convert(a.p, dt);
  V dv = t.dot(pd, g, {0, 1}, {0, 1}, {2}, {2}, grouped ? DType::F32 : dt);                 // [B, N, S, H]
  V dp = t.dot(g, a.v, {0, 1}, {0, 1}, {3}, {3}, DType::F32);                                // [B, N, T, S]
  V ds = t.mul(a.p, t.sub(dp, t.reduceBack("add", t.mul(dp, a.p), {3}, 0.0)));
  V dsd = t.convert(t.mulc(ds, scale), dt);
  V dq = t.dot(dsd, a.k, {0, 1}, {0, 1}, {3}, {2}, dt);                                      // [B, N, T, H]
  V dk = t.dot(dsd, a.q, {0, 1}, {0, 1}, {2}, {2}, grouped ? DType::F32 : dt);               // [B, N, S, H]
  if (grouped) {       // the heads that shared a key / value head add up
    const int64_t grp = a.N / a.Nkv;
    auto fold = [&](const V& x) { return t.convert(t.reduce("add", t.reshape(x, {a.B, a.Nkv, grp, a.S, a.H}), {2}, 0.0), dt); };
    dk = fold(dk);
    dv = fold(dv);
  }
  return t.function(fn, {dq, dk, dv});
}

// ---- normalisations over the last dim -------------------------------------------------------------------------------
std::vector<int64_t> leadingDims(const TensorType& x) {
  std::vector<int64_t> d;
  for (int k = 0; k + 1 < x.rank(); ++k) d.push_back(k);
  return d;
}

void checkRowOperand(const std::string& target, const TensorType& x, const TensorType& w, const char* what) {
  if (!isFloat(x.dt) || x.rank() < 1) bad(target, "the input must be a float tensor with at least one dim");
  if (w.rank() != 1 || w.dims[0] != x.dims.back() || w.dt != x.dt) bad(target, std::string(what) + " must be one-dimensional, of the input's last dim and type");
}

std::string rmsNorm(const std::string& target, const std::string& fn, const std::vector<TensorType>& in, bool backward, const Config& c) {
  checkRowOperand(target, in[0], in[1], "the weight");
  Text t;
  V x = t.arg(in[0]), w = t.arg(in[1]);
  const double eps = c.number("eps", 1e-6);
  V x32 = t.convert(x, DType::F32), w32 = t.bcastTo(t.convert(w, DType::F32), x.t.dims);
  V r = t.unary("rsqrt", t.addc(t.rowMean(t.mul(x32, x32)), eps));
  V xn = t.mul(x32, r);
  if (!backward) return t.function(fn, {t.convert(t.mul(xn, w32), x.t.dt)});
  V g = t.arg(in[2]);
  if (!(g.t == x.t)) bad(target, "the output gradient must have the input's type");
  V g32 = t.convert(g, DType::F32);
  V gw = t.mul(g32, w32);
  V dx = t.mul(r, t.sub(gw, t.mul(xn, t.rowMean(t.mul(gw, xn)))));
  V dw = t.reduce("add", t.mul(g32, xn), leadingDims(x.t), 0.0);
  return t.function(fn, {t.convert(dx, x.t.dt), t.convert(dw, w.t.dt)});
}

std::string layerNorm(const std::string& target, const std::string& fn, const std::vector<TensorType>& in, bool backward, const Config& c) {
  checkRowOperand(target, in[0], in[1], "the weight");
  checkRowOperand(target, in[0], in[2], "the bias");
  Text t;
  V x = t.arg(in[0]), w = t.arg(in[1]), b = t.arg(in[2]);
  const double eps = c.number("eps", 1e-5);
  V x32 = t.convert(x, DType::F32), w32 = t.bcastTo(t.convert(w, DType::F32), x.t.dims);
  V d = t.sub(x32, t.rowMean(x32));
  V r = t.unary("rsqrt", t.addc(t.rowMean(t.mul(d, d)), eps));
  V xn = t.mul(d, r);
  if (!backward) return t.function(fn, {t.convert(t.add(t.mul(xn, w32), t.bcastTo(t.convert(b, DType::F32), x.t.dims)), x.t.dt)});
  V g = t.arg(in[3]);
  if (!(g.t == x.t)) bad(target, "the output gradient must have the input's type");
  V g32 = t.convert(g, DType::F32);
  V gw = t.mul(g32, w32);
  V dx = t.mul(r, t.sub(t.sub(gw, t.rowMean(gw)), t.mul(xn, t.rowMean(t.mul(gw, xn)))));
  V dw = t.reduce("add", t.mul(g32, xn), leadingDims(x.t), 0.0);
  V db = t.reduce("add", g32, leadingDims(x.t), 0.0);
  return t.function(fn, {t.convert(dx, x.t.dt), t.convert(dw, w.t.dt), t.convert(db, b.t.dt)});
}

// ---- rotary position embedding -------------------------------------------------------------------------------------
// x is (..., T, D); the first `dims` features rotate by angle (position + offset) * rope_scale * base^(-2i / dims), as
// halves (x[i], x[i + dims/2]) or, "traditional", as neighbouring pairs (x[2i], x[2i+1]); the backward form applies the
// inverse rotation to the gradient (the map is linear and orthogonal per pair).
std::string rope(const std::string& target, const std::string& fn, const std::vector<TensorType>& in, bool backward, const Config& c) {
  const TensorType& xt = in[0];
  if (!isFloat(xt.dt) || xt.rank() < 2) bad(target, "the input must be a float tensor (..., T, D)");
  if (in[1].numel() != 1 || !(isInt(in[1].dt) || isFloat(in[1].dt))) bad(target, "the offset must be one number");
  const int64_t D = xt.dims.back(), T = xt.dims[(size_t)xt.rank() - 2];
  const int64_t dims = (int64_t)c.number("dims", (double)D);
  if (dims <= 0 || dims > D || dims % 2) bad(target, "dims must be even and at most the last dim");
  const bool traditional = c.boolean("traditional", false);
  const double base = c.number("base", 10000.0), ropeScale = c.number("rope_scale", 1.0);
  const int64_t half = dims / 2;
  Text t;
  V x = t.arg(xt), offset = t.arg(in[1]);
  V src = x;
  if (backward) {
    src = t.arg(in[2]);
    if (!(src.t == xt)) bad(target, "the output gradient must have the input's type");
  }
  const int last = xt.rank() - 1;
  // angles[t, i], float32
  V pos = t.convert(t.iota(DType::S32, {T, half}, 0), DType::F32);
  V off = t.bcast(t.reshape(t.convert(offset, DType::F32), {}), {T, half}, {});
  pos = t.mulc(t.add(pos, off), ropeScale);
  V idx = t.convert(t.iota(DType::S32, {T, half}, 1), DType::F32);
  V freq = t.unary("exponential", t.mulc(idx, -2.0 * std::log(base) / (double)dims));
  V ang = t.mul(pos, freq);
  std::vector<int64_t> halfShape = xt.dims;
  halfShape[(size_t)last] = half;
  const std::vector<int64_t> tail = {(int64_t)xt.rank() - 2, (int64_t)xt.rank() - 1};
  V cosv = t.bcast(t.unary("cosine", ang), halfShape, tail);
  V sinv = t.bcast(t.unary("sine", ang), halfShape, tail);
  if (backward) sinv = t.unary("negate", sinv);
  V s32 = t.convert(src, DType::F32);
  V a, b;
  if (traditional) { a = t.slice(s32, last, 0, dims, 2); b = t.slice(s32, last, 1, dims, 2); }
  else { a = t.slice(s32, last, 0, half); b = t.slice(s32, last, half, dims); }
  V ra = t.sub(t.mul(a, cosv), t.mul(b, sinv));
  V rb = t.add(t.mul(b, cosv), t.mul(a, sinv));
  V rot;
  if (traditional) {
    std::vector<int64_t> pairShape = halfShape;
    pairShape.push_back(1);
    V both = t.concat({t.reshape(ra, pairShape), t.reshape(rb, pairShape)}, last + 1);
    std::vector<int64_t> flat = xt.dims;
    flat[(size_t)last] = dims;
    rot = t.reshape(both, flat);
  } else {
    rot = t.concat({ra, rb}, last);
  }
  V out = t.convert(rot, xt.dt);
  if (dims < D) out = t.concat({out, t.slice(src, last, dims, D)}, last);
  return t.function(fn, {out});
}

// ---- gelu (tanh form) ----------------------------------------------------------------------------------------------
std::string gelu(const std::string& target, const std::string& fn, const std::vector<TensorType>& in, bool backward) {
  if (!isFloat(in[0].dt)) bad(target, "the input must be a float tensor");
  Text t;
  V x = t.arg(in[0]);
  const double c0 = 0.7978845608028654, c1 = 0.044715;
  V x32 = t.convert(x, DType::F32);
  V x2 = t.mul(x32, x32);
  V th = t.unary("tanh", t.mulc(t.add(x32, t.mulc(t.mul(x2, x32), c1)), c0));
  if (!backward) return t.function(fn, {t.convert(t.mul(t.mulc(x32, 0.5), t.addc(th, 1.0)), x.t.dt)});
  V g = t.arg(in[1]);
  if (!(g.t == x.t)) bad(target, "the output gradient must have the input's type");
  // d/dx [0.5 x (1 + tanh u)] = 0.5 (1 + tanh u) + 0.5 x (1 - tanh^2 u) c0 (1 + 3 c1 x^2)
  V sech2 = t.sub(t.splat(1.0, th.t), t.mul(th, th));
  V du = t.mulc(t.addc(t.mulc(x2, 3.0 * c1), 1.0), c0);
  V d = t.add(t.mulc(t.addc(th, 1.0), 0.5), t.mul(t.mulc(x32, 0.5), t.mul(sech2, du)));
  return t.function(fn, {t.convert(t.mul(t.convert(g, DType::F32), d), x.t.dt)});
}

struct Target {
  const char* name;
  int operands, results;
};
const Target kTargets[] = {{"sdpa", 4, 1},      {"sdpa_causal", 3, 1},    {"sdpa_bwd", 5, 3}, {"sdpa_causal_bwd", 4, 3}, {"rms_norm", 2, 1}, {"rms_norm_bwd", 3, 2},
                           {"layer_norm", 3, 1}, {"layer_norm_bwd", 4, 3}, {"rope", 2, 1},     {"rope_bwd", 3, 1},        {"gelu", 1, 1},     {"gelu_bwd", 2, 1}};

void lowerIn(Module& m, Region& r, int& serial) {
  for (auto& o : r.ops) {
    for (auto& sub : o->regions) lowerIn(m, *sub, serial);
    if (o->name != "custom_call") continue;
    const std::string target = o->str("target");
    std::string op;
    if (target.rfind("mps.", 0) == 0) op = target.substr(4);
    else if (target.rfind("mi355x.", 0) == 0) op = target.substr(7);
    else continue;
    const Target* known = nullptr;
    for (auto& t : kTargets) if (op == t.name) known = &t;
    if (!known) continue;          // left for the supported-op check, which names it
    if ((int)o->operands.size() != known->operands || (int)o->results.size() != known->results)
      bad(target, "expected " + std::to_string(known->operands) + " inputs and " + std::to_string(known->results) + " outputs");
    std::vector<TensorType> in;
    for (auto* v : o->operands) in.push_back(v->type);
    Config cfg{o->str("backend_config")};
    const std::string fn = "__fused_" + op + "_" + std::to_string(serial++);
    std::string text;
    if (op == "sdpa") text = sdpaForward(target, fn, in, false, cfg);
    else if (op == "sdpa_causal") text = sdpaForward(target, fn, in, true, cfg);
    else if (op == "sdpa_bwd") text = sdpaBackward(target, fn, in, false, cfg);
    else if (op == "sdpa_causal_bwd") text = sdpaBackward(target, fn, in, true, cfg);
    else if (op == "rms_norm" || op == "rms_norm_bwd") text = rmsNorm(target, fn, in, op == "rms_norm_bwd", cfg);
    else if (op == "layer_norm" || op == "layer_norm_bwd") text = layerNorm(target, fn, in, op == "layer_norm_bwd", cfg);
    else if (op == "rope" || op == "rope_bwd") text = rope(target, fn, in, op == "rope_bwd", cfg);
    else text = gelu(target, fn, in, op == "gelu_bwd");
    std::unique_ptr<Module> piece;
    try {
      piece = parseStableHLOText(text.data(), text.size());
    } catch (const CompileError& e) {
      throw CompileError("internal: the expansion of custom_call @" + target + " does not parse: " + e.what() + "\n" + text);
    }
    Func* f = piece->funcs.size() == 1 ? piece->funcs[0].get() : nullptr;     // (the front end names a lone function "main")
    if (f) f->name = fn;
    if (!f || f->resultTypes.size() != o->results.size()) throw CompileError("internal: the expansion of custom_call @" + target + " is malformed");
    for (size_t k = 0; k < o->results.size(); ++k)
      if (!(f->resultTypes[k] == o->results[k]->type))
        bad(target, "result " + std::to_string(k) + " is declared " + o->results[k]->type.str() + " but the operation yields " + f->resultTypes[k].str());
    for (auto& pf : piece->funcs) m.funcs.push_back(std::move(pf));
    o->name = "call";
    Attr callee;
    callee.kind = Attr::Str;
    callee.s = fn;
    o->attrs.clear();
    o->attrs["callee"] = callee;
  }
}

}  // namespace

void lowerFusedOpCalls(Module& m) {
  int serial = 0;
  const size_t n = m.funcs.size();          // functions appended by the rewrite hold no custom calls
  for (size_t k = 0; k < n; ++k) lowerIn(m, m.funcs[k]->body, serial);
}

}  // namespace mi355
