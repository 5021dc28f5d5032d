// Generator of fused HIP kernels (loop fusion, dynamic_update_slice windows and
// reductions).  Every generated kernel is built from the same hand-written
// skeletons below: a streaming skeleton that moves 16 bytes per lane with
// vector loads/stores, a row-reduction skeleton (lanes along the reduced,
// contiguous axis; wavefront shuffles then one LDS step) and a column-reduction
// skeleton (lanes along the kept, contiguous axis; LDS step across row groups;
// optional second pass over partials).  Only the per-element expression inside
// the skeleton is produced from the StableHLO ops.
//
// Op semantics follow the reference's handlers: ops/arithmetic.cc:535-607
// (elementwise, compare, shifts, remainder, integer divide, sign, rounding),
// ops/shape.cc:260-270, ops/slice.cc:90-276 (clamped dynamic starts, pad),
// ops/gather_scatter.cc:200-294 (gather with clamped starts),
// ops/reduction.cc:83-162 (reduce by body pattern).
#include "codegen.h"

#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <numeric>
#include <sstream>
#include <memory>
#include <unordered_map>
#include <unordered_set>

namespace mi355 {

namespace {

const char* kPrelude = R"HIP(
typedef unsigned short u16; typedef unsigned int u32; typedef unsigned long long u64; typedef long long i64;
typedef signed char i8; typedef unsigned char u8; typedef short i16;
template <typename T, int N> struct __attribute__((aligned(sizeof(T) * N))) Vec { T e[N]; };
__device__ __forceinline__ float bf2f(u16 b) { return __uint_as_float(((u32)b) << 16); }
// gfx950 rounds f32 -> bf16 (nearest even, NaN stays NaN) in one instruction
__device__ __forceinline__ u16 f2bf(float f) { return __builtin_bit_cast(u16, (__bf16)f); }
__device__ __forceinline__ float bfr(float f) { return bf2f(f2bf(f)); }
// f32 -> f16 of a value that exists as an f32 first: without the empty statement the compiler folds a product and its
// narrowing into one mixed-precision multiply-add with a +0 addend, which rounds once and turns a product of -0 into +0
__device__ __forceinline__ _Float16 f2h(float f) { asm volatile("" : "+v"(f)); return (_Float16)f; }
__device__ __forceinline__ float hfr(float f) { return (float)f2h(f); }
template <typename T> __device__ __forceinline__ T mx(T a, T b) { return (a > b || a != a) ? a : b; }
template <typename T> __device__ __forceinline__ T mn(T a, T b) { return (a < b || a != a) ? a : b; }
template <typename I, typename F> __device__ __forceinline__ I f2i(F f) {
  if (f != f) return (I)0;
  const bool sg = (I)(-1) < (I)0;
  const int bits = (int)sizeof(I) * 8;
  const F hi = sg ? (F)(1ull << (bits - 1)) : (bits == 64 ? (F)18446744073709551615.0 : (F)(1ull << (bits & 63)));
  if (f >= hi) return sg ? (I)((1ull << (bits - 1)) - 1ull) : (I)~(I)0;
  if (sg) { if (f <= -hi) return (I)(1ull << (bits - 1)); }
  else if (f <= (F)0) return (I)0;
  return (I)f;
}
// Integer arithmetic wraps (two's complement), for signed types as well: the 32- and 64-bit ones are computed on their
// unsigned counterparts, where overflow is defined (narrower types are promoted to int by the language and wrap when
// they are narrowed again).
template <typename T> struct Uns { typedef T type; };
template <> struct Uns<int> { typedef u32 type; };
template <> struct Uns<i64> { typedef u64 type; };
template <typename T> __device__ __forceinline__ T wadd(T a, T b) { typedef typename Uns<T>::type U; return (T)((U)a + (U)b); }
template <typename T> __device__ __forceinline__ T wsub(T a, T b) { typedef typename Uns<T>::type U; return (T)((U)a - (U)b); }
template <typename T> __device__ __forceinline__ T wmul(T a, T b) { typedef typename Uns<T>::type U; return (T)((U)a * (U)b); }
template <typename T> __device__ __forceinline__ T ipow(T a, T b) {
  if (b < (T)0) return a == (T)1 ? (T)1 : (a == (T)-1 ? ((b & (T)1) ? (T)-1 : (T)1) : (T)0);
  T r = (T)1;
  while (b) { if (b & (T)1) r = wmul<T>(r, a); a = wmul<T>(a, a); b >>= 1; }
  return r;
}
// division by zero gives all ones, the most negative number divided by -1 itself (and remainder 0); an unsigned divisor
// of all ones is an ordinary number
template <typename T> __device__ __forceinline__ T idiv(T a, T b) {
  const bool sg = (T)-1 < (T)0;
  return b == (T)0 ? (T)-1 : ((sg && b == (T)-1) ? wsub<T>((T)0, a) : (T)(a / b));
}
template <typename T> __device__ __forceinline__ T irem(T a, T b) {
  const bool sg = (T)-1 < (T)0;
  return b == (T)0 ? a : ((sg && b == (T)-1) ? (T)0 : (T)(a % b));
}
// 16-bit results keep 8 (bf16) or 11 (f16) significand bits: the hardware exponential is exact enough there
// (near zero 1 - exp cancels; below 4e-4 the argument itself is the result to 5e-8 relative, and from there on the
// difference still holds the 11 bits a 16-bit result keeps)
__device__ __forceinline__ float tanh_fast(float x) {
  float t = __expf(-2.f * fabsf(x));
  float r = copysignf((1.f - t) * __builtin_amdgcn_rcpf(1.f + t), x);
  return fabsf(x) < 4e-4f ? x : r;
}
// the same where only the absolute error counts (1 + tanh(u) of a GELU): no special case near zero
__device__ __forceinline__ float tanh_fast_abs(float x) { float t = __expf(-2.f * fabsf(x)); return copysignf((1.f - t) * __builtin_amdgcn_rcpf(1.f + t), x); }
// f32 tanh to a few ulp: odd polynomial near 0 (where 1 - exp cancels), exponential form elsewhere
__device__ __forceinline__ float tanh_f32(float x) {
  float ax = fabsf(x), x2 = x * x;
  float p = x * (1.f + x2 * (-0.33333334f + x2 * (0.13333334f + x2 * (-0.05396825f + x2 * (0.021869488f + x2 * -0.008863236f)))));
  float t = __expf(-2.f * ax);
  float r = copysignf((1.f - t) * __builtin_amdgcn_rcpf(1.f + t), x);
  return ax < 0.3f ? p : r;
}
__device__ __forceinline__ float sgnf(float x) { return (x != x || x == 0.f) ? x : (x > 0.f ? 1.f : -1.f); }
__device__ __forceinline__ double sgnd(double x) { return (x != x || x == 0.0) ? x : (x > 0.0 ? 1.0 : -1.0); }
__device__ __forceinline__ int tokey(float f) { int i = __float_as_int(f); return i < 0 ? (i ^ 0x7FFFFFFF) : i; }
__device__ __forceinline__ float redprec(float x, int eb, int mb) {
  u32 u = __float_as_uint(x);
  if (mb < 23 && x == x) { int sh = 23 - mb; u32 lsb = (u >> sh) & 1u; u = (u + ((1u << (sh - 1)) - 1u) + lsb) & ~((1u << sh) - 1u); }
  float y = __uint_as_float(u);
  if (eb < 8 && x == x) {
    int maxe = (1 << (eb - 1)) - 1, mine = 1 - maxe;
    int e = (int)((u >> 23) & 0xFF) - 127;
    bool neg = (u >> 31) != 0;
    if (e > maxe && e != 128) y = neg ? -__builtin_inff() : __builtin_inff();
    if (e < mine) y = neg ? -0.f : 0.f;
  }
  return y;
}
)HIP";

std::string storageT(DType d) {
  switch (d) {
    case DType::F32: return "float";
    case DType::F64: return "double";
    case DType::F16: return "_Float16";
    case DType::BF16: return "u16";
    case DType::S8: return "i8";
    case DType::U8: return "u8";
    case DType::Pred: return "u8";
    case DType::S16: return "i16";
    case DType::U16: return "u16";
    case DType::S32: return "int";
    case DType::U32: return "u32";
    case DType::S64: return "i64";
    case DType::U64: return "u64";
    default: throw CompileError("codegen: unsupported element type");
  }
}
std::string computeT(DType d) {
  switch (d) {
    case DType::F32: case DType::F16: case DType::BF16: return "float";
    case DType::F64: return "double";
    case DType::Pred: return "bool";
    default: return storageT(d);
  }
}
std::string loadExpr(DType d, const std::string& e) {
  if (d == DType::BF16) return "bf2f(" + e + ")";
  if (d == DType::F16) return "(float)(" + e + ")";
  if (d == DType::Pred) return "((" + e + ") != 0)";
  return e;
}
std::string storeExpr(DType d, const std::string& e) {
  if (d == DType::BF16) return "f2bf(" + e + ")";
  if (d == DType::F16) return "f2h(" + e + ")";
  if (d == DType::Pred) return "(u8)((" + e + ") ? 1 : 0)";
  return e;
}
std::string roundTo(DType d, const std::string& e) {
  if (d == DType::BF16) return "bfr(" + e + ")";
  if (d == DType::F16) return "hfr(" + e + ")";
  return e;
}

std::string literalFromBytes(DType d, const uint8_t* p) {
  char buf[64];
  switch (d) {
    case DType::F32: { uint32_t u; memcpy(&u, p, 4); snprintf(buf, sizeof buf, "__uint_as_float(0x%08xu)", u); return buf; }
    case DType::BF16: { uint16_t h; memcpy(&h, p, 2); snprintf(buf, sizeof buf, "__uint_as_float(0x%08xu)", ((uint32_t)h) << 16); return buf; }
    case DType::F16: { _Float16 h; memcpy(&h, p, 2); float f = (float)h; uint32_t u; memcpy(&u, &f, 4); snprintf(buf, sizeof buf, "__uint_as_float(0x%08xu)", u); return buf; }
    case DType::F64: { uint64_t u; memcpy(&u, p, 8); snprintf(buf, sizeof buf, "__longlong_as_double(0x%016llxll)", (unsigned long long)u); return buf; }
    case DType::Pred: return *p ? "true" : "false";
    case DType::S8: snprintf(buf, sizeof buf, "(i8)%d", (int)*(const int8_t*)p); return buf;
    case DType::U8: snprintf(buf, sizeof buf, "(u8)%u", (unsigned)*p); return buf;
    case DType::S16: { int16_t v; memcpy(&v, p, 2); snprintf(buf, sizeof buf, "(i16)%d", (int)v); return buf; }
    case DType::U16: { uint16_t v; memcpy(&v, p, 2); snprintf(buf, sizeof buf, "(u16)%u", (unsigned)v); return buf; }
    case DType::S32: { int32_t v; memcpy(&v, p, 4); if (v == INT32_MIN) return "(-2147483647 - 1)"; snprintf(buf, sizeof buf, "%d", v); return buf; }
    case DType::U32: { uint32_t v; memcpy(&v, p, 4); snprintf(buf, sizeof buf, "%uu", v); return buf; }
    case DType::S64: { int64_t v; memcpy(&v, p, 8); if (v == INT64_MIN) return "(-9223372036854775807ll - 1)"; snprintf(buf, sizeof buf, "%lldll", (long long)v); return buf; }
    case DType::U64: { uint64_t v; memcpy(&v, p, 8); snprintf(buf, sizeof buf, "%lluull", (unsigned long long)v); return buf; }
    default: throw CompileError("codegen: literal of unsupported type");
  }
}

int64_t gcd64(int64_t a, int64_t b) {
  a = a < 0 ? -a : a;
  b = b < 0 ? -b : b;
  while (b) { int64_t t = a % b; a = b; b = t; }
  return a;
}

// One index component: value = base + coef * v, where v is the lane number inside the thread's vector.
struct IdxDim {
  std::string base = "0";
  int64_t coef = 0;
  bool inBody = false;   // base is a variable of the per-lane loop body
  bool isConst = true;
  int64_t cval = 0;
  int64_t mult = 0;      // base is a known multiple of `mult` (0 = the constant zero, divisible by anything)
  bool lane() const { return inBody || coef != 0; }
};

IdxDim constDim(int64_t c) {
  IdxDim d;
  d.base = std::to_string(c);
  d.isConst = true;
  d.cval = c;
  d.mult = c;
  return d;
}

struct Index {
  bool linear = false;
  IdxDim lin;
  std::vector<int64_t> shape;   // shape the index addresses
  std::vector<IdxDim> dims;     // valid when !linear
  std::string sig;              // structural signature for memoisation
  bool lane() const {
    if (linear) return lin.lane();
    for (auto& d : dims) if (d.lane()) return true;
    return false;
  }
};

class Emitter {
 public:
  Emitter(const LeafPredicate& isLeaf, int V, bool idx64) : V_(V), idx64_(idx64), isLeaf_(isLeaf) {
    body_.emplace_back();
    cache_.emplace_back();
  }

  int V_;
  bool idx64_;
  std::string pre_;
  std::vector<std::string> body_;
  std::vector<Value*> leaves_;

  std::string idxT() const { return idx64_ ? "i64" : "int"; }
  std::string fresh(const char* p) { return std::string(p) + std::to_string(tmp_++); }
  void pre(const std::string& s) { pre_ += "  " + s + "\n"; }
  void body(const std::string& s) { body_.back() += std::string(2 + 2 * body_.size(), ' ') + s + "\n"; }
  void emit(bool inBody, const std::string& s) { (inBody || guard_ > 0) ? body(s) : pre(s); }

  // Names declared inside the lane loop.  An expression that mentions one of them has to be emitted
  // there too, whatever its index looks like (with one element per lane nothing is lane-dependent
  // by index, yet guarded loads, concatenations and their consumers still live in the loop body).
  std::unordered_set<std::string> bodyNames_;
  bool mentionsBody(const std::string& e) const {
    if (bodyNames_.empty()) return false;
    size_t i = 0, n = e.size();
    while (i < n) {
      if (isalpha((unsigned char)e[i]) || e[i] == '_') {
        size_t j = i;
        while (j < n && (isalnum((unsigned char)e[j]) || e[j] == '_')) ++j;
        if (bodyNames_.count(e.substr(i, j - i))) return true;
        i = j;
      } else {
        ++i;
      }
    }
    return false;
  }

  // Row programs: results of reductions finished earlier in the same kernel, as variables that
  // hold the value for the row this wavefront / workgroup owns.
  std::unordered_map<Value*, std::string> rowScalars_;
  std::unordered_map<std::string, std::string> rowRcp_;   // row scalar variable -> variable holding its reciprocal
  std::vector<IdxDim> rowKept_;           // index of the current row over the kept dims
  // Row programs with unrolled walks: values an earlier walk computed at the same element, as the
  // expression that reads them back from the registers they were kept in.  A lookup that lands on one
  // stops there (the walk is top-down, so the hits are the values closest to the roots) and is recorded.
  std::unordered_map<std::string, std::string> seeded_;
  std::unordered_set<std::string> seededUsed_;
  int seededCap_ = 0;
  std::unordered_map<std::string, Value*> keyValue_;
  const std::unordered_map<std::string, std::string>& unguardedValues() const { return cache_.front(); }
  void shareLeavesFrom(const Emitter& o) { leaves_ = o.leaves_; leafIndex_ = o.leafIndex_; }
  void startTemporariesAt(int n) { tmp_ = n; }   // keeps the names of nested emitters apart

  int leafId(Value* v) {
    auto it = leafIndex_.find(v);
    if (it != leafIndex_.end()) return it->second;
    int id = (int)leaves_.size();
    leaves_.push_back(v);
    leafIndex_[v] = id;
    return id;
  }

  std::string dimExpr(const IdxDim& d) const {
    if (d.isConst) return d.base;
    if (d.inBody || d.coef == 0) return d.base;
    if (d.coef == 1) return "(" + d.base + " + v)";
    return "(" + d.base + " + " + std::to_string(d.coef) + " * v)";
  }

  // new index variable holding `expr`
  IdxDim var(const std::string& expr, bool inBody, int64_t coef = 0, int64_t mult = 1) {
    IdxDim d;
    d.isConst = false;
    const bool forced = !inBody && mentionsBody(expr);
    d.inBody = inBody || guard_ > 0 || forced;
    d.base = fresh("ix");
    d.coef = d.inBody ? 0 : coef;
    d.mult = mult;
    // a lane-dependent value (expr + coef * v) that is forced into the lane loop by a guarded scope
    // becomes a plain per-lane variable: its lane term has to be part of the expression
    const std::string full = (!inBody && (guard_ > 0 || forced) && coef != 0) ? "(" + expr + " + " + std::to_string(coef) + " * v)" : expr;
    emit(d.inBody, "const " + idxT() + " " + d.base + " = " + full + ";");
    if (d.inBody) bodyNames_.insert(d.base);
    return d;
  }

  IdxDim toBody(const IdxDim& d) {
    if (d.isConst || d.inBody) return d;
    if (d.coef == 0 && guard_ == 0) return d;
    IdxDim r;
    r.isConst = false;
    r.inBody = true;
    r.base = fresh("ix");
    bodyNames_.insert(r.base);
    body("const " + idxT() + " " + r.base + " = " + dimExpr(d) + ";");
    return r;
  }

  // a*d + c
  IdxDim affine(const IdxDim& d, int64_t a, int64_t c) {
    if (d.isConst) return constDim(a * d.cval + c);
    if (a == 1 && c == 0) return d;
    if (d.inBody) return var("(" + d.base + " * " + std::to_string(a) + " + " + std::to_string(c) + ")", true);
    std::string e = a == 1 ? d.base : "(" + d.base + " * " + std::to_string(a) + ")";
    if (c != 0) e = "(" + e + " + " + std::to_string(c) + ")";
    int64_t m = gcd64(d.mult * a, c);
    return var(e, false, d.coef * a, m == 0 ? 1 : m);
  }

  IdxDim addDims(const IdxDim& a, const IdxDim& b) {
    if (a.isConst) return affine(b, 1, a.cval);
    if (b.isConst) return affine(a, 1, b.cval);
    if (a.inBody || b.inBody) return var("(" + dimExpr(a) + " + " + dimExpr(b) + ")", true);
    return var("(" + a.base + " + " + b.base + ")", false, a.coef + b.coef, std::max<int64_t>(1, gcd64(a.mult, b.mult)));
  }

  std::vector<IdxDim> delinearize(IdxDim lin, const std::vector<int64_t>& shape) {
    int n = (int)shape.size();
    std::vector<IdxDim> out(n);
    if (n == 0) return out;
    if (lin.isConst) {
      int64_t r = lin.cval;
      for (int d = n - 1; d >= 0; --d) {
        int64_t D = std::max<int64_t>(shape[d], 1);
        out[d] = constDim(d == 0 ? r : r % D);
        r /= D;
      }
      return out;
    }
    int last = n - 1;
    if (!lin.inBody && lin.coef != 0) {
      int64_t D = shape[last];
      bool ok = lin.coef == 1 && D % V_ == 0 && lin.mult % V_ == 0;
      if (!ok) lin = toBody(lin);
      else {
        if (n == 1) { out[0] = lin; return out; }
        out[last] = var("(" + lin.base + " % " + std::to_string(D) + ")", false, 1, V_);
        IdxDim rest = var("(" + lin.base + " / " + std::to_string(D) + ")", false, 0, 1);
        auto head = delinearize(rest, std::vector<int64_t>(shape.begin(), shape.begin() + last));
        for (int d = 0; d < last; ++d) out[d] = head[d];
        return out;
      }
    }
    // lane-invariant or per-lane scalar: plain div/mod chain
    bool inB = lin.inBody;
    std::string rem = lin.base;
    for (int d = n - 1; d >= 0; --d) {
      int64_t D = shape[d];
      if (D == 1) { out[d] = constDim(0); continue; }
      bool anyLeft = false;
      for (int q = 0; q < d; ++q) if (shape[q] != 1) anyLeft = true;
      if (!anyLeft) { IdxDim r; r.isConst = false; r.inBody = inB; r.base = rem; r.mult = 1; out[d] = r; for (int q = 0; q < d; ++q) out[q] = constDim(0); break; }
      out[d] = var("(" + rem + " % " + std::to_string(D) + ")", inB);
      IdxDim q = var("(" + rem + " / " + std::to_string(D) + ")", inB);
      rem = q.base;
    }
    return out;
  }

  IdxDim linearize(const std::vector<IdxDim>& dims, const std::vector<int64_t>& shape) {
    int n = (int)shape.size();
    std::vector<int64_t> stride(n, 1);
    for (int d = n - 2; d >= 0; --d) stride[d] = stride[d + 1] * shape[d + 1];
    // inside a guarded scope every new index variable lives in the lane loop, so the per-lane
    // term of each component has to be spelled out
    bool anyBody = guard_ > 0, allConst = true;
    int64_t cst = 0;
    for (int d = 0; d < n; ++d) {
      if (dims[d].isConst) cst += dims[d].cval * stride[d];
      else { allConst = false; if (dims[d].inBody) anyBody = true; }
    }
    if (allConst) return constDim(cst);
    std::string e;
    int64_t coef = 0, mult = cst;
    int terms = 0;
    const IdxDim* single = nullptr;
    for (int d = 0; d < n; ++d) {
      if (dims[d].isConst) continue;
      std::string t = anyBody ? dimExpr(dims[d]) : dims[d].base;
      if (stride[d] != 1) t = t + " * " + std::to_string(stride[d]);
      e += (e.empty() ? "" : " + ") + t;
      coef += dims[d].coef * stride[d];
      mult = gcd64(mult, dims[d].mult * stride[d]);
      ++terms;
      if (stride[d] == 1) single = &dims[d];
    }
    if (terms == 1 && cst == 0 && single) return *single;
    if (cst != 0) e += " + " + std::to_string(cst);
    if (anyBody) return var("(" + e + ")", true);
    return var("(" + e + ")", false, coef, mult == 0 ? 1 : mult);
  }

  Index multi(const Index& idx) {
    if (!idx.linear) return idx;
    Index m;
    m.linear = false;
    m.shape = idx.shape;
    m.dims = delinearize(idx.lin, idx.shape);
    finishSig(m);
    return m;
  }

  void finishSig(Index& idx) {
    std::string s;
    if (idx.linear) s = "L" + idx.lin.base + "#" + std::to_string(idx.lin.coef);
    else for (auto& d : idx.dims) s += d.base + "#" + std::to_string(d.coef) + ",";
    idx.sig = s;
  }

  Index linearIndex(const IdxDim& lin, const std::vector<int64_t>& shape) {
    Index i;
    i.linear = true;
    i.lin = lin;
    i.shape = shape;
    finishSig(i);
    return i;
  }
  Index multiIndex(std::vector<IdxDim> dims, const std::vector<int64_t>& shape) {
    Index i;
    i.linear = false;
    i.dims = std::move(dims);
    i.shape = shape;
    finishSig(i);
    return i;
  }

  // ----------------------------------------------------------------- loads
  std::string load(Value* leaf, const Index& idx) {
    int id = leafId(leaf);
    DType dt = leaf->type.dt;
    std::string ptr = "in" + std::to_string(id);
    IdxDim off = idx.linear ? idx.lin : linearize(idx.dims, leaf->type.dims);
    bool inB = off.inBody || guard_ > 0;
    if (!inB && off.coef == 1 && V_ > 1 && !off.isConst && off.mult % V_ == 0 && leaf->type.numel() % V_ == 0) {
      // one aligned vector load per thread, hoisted out of the lane loop
      std::string key = ptr + "@" + off.base;
      auto it = vecLoads_.find(key);
      std::string name;
      if (it == vecLoads_.end()) {
        name = fresh("lv");
        pre("const Vec<" + storageT(dt) + ", " + std::to_string(V_) + "> " + name + " = *(const Vec<" + storageT(dt) + ", " +
            std::to_string(V_) + ">*)(" + ptr + " + " + off.base + ");");
        vecLoads_[key] = name;
      } else {
        name = it->second;
      }
      return loadExpr(dt, name + ".e[v]");
    }
    std::string t = fresh("ld");
    if (!inB && off.coef == 0) {
      pre("const " + computeT(dt) + " " + t + " = " + loadExpr(dt, ptr + "[" + (off.isConst ? off.base : off.base) + "]") + ";");
      return t;
    }
    bodyNames_.insert(t);
    body("const " + computeT(dt) + " " + t + " = " + loadExpr(dt, ptr + "[" + dimExpr(off) + "]") + ";");
    return t;
  }

  // What was declared inside a loop body that has been written out is out of scope for the code that follows it.
  void forgetBodyValues() {
    for (auto& c : cache_)
      for (auto it = c.begin(); it != c.end();) it = bodyNames_.count(it->second) ? c.erase(it) : std::next(it);
  }

  // --------------------------------------------------------- value generation
  std::string gen(Value* v, const Index& idx) {
    std::string key = std::to_string(v->id) + "|" + idx.sig;
    for (int s = (int)cache_.size() - 1; s >= 0; --s) {
      auto it = cache_[s].find(key);
      if (it != cache_[s].end()) return it->second;
    }
    if (!seeded_.empty()) {
      auto sd = seeded_.find(key);
      if (sd != seeded_.end() && (seededUsed_.count(key) || (int)seededUsed_.size() < seededCap_)) {
        seededUsed_.insert(key);
        return sd->second;
      }
    }
    keyValue_[key] = v;
    std::string r = genUncached(v, idx);
    // values emitted into the lane-invariant prologue are visible everywhere
    bool laneInv = !idx.lane() && guard_ == 0;
    (laneInv ? cache_.front() : cache_.back())[key] = r;
    return r;
  }

 private:
  const LeafPredicate& isLeaf_;
  int tmp_ = 0;
  int guard_ = 0;
  std::unordered_map<Value*, int> leafIndex_;
  std::unordered_map<std::string, std::string> vecLoads_;
  std::vector<std::unordered_map<std::string, std::string>> cache_;

  // 16-bit float results are computed in fp32.  Inside a fused chain they are rounded to their
  // own precision only where the program asks for the narrowing (convert and friends) or where
  // they are stored; rounding after every arithmetic op (MI355X_STRICT_BF16=1) costs two
  // instructions per op and only loses accuracy.  The switch is read at every compile, like the
  // reference's JAX_MPS_NO_OPTIMIZE (stablehlo_parser.cc:83-85), so one process can hold programs of both kinds.
  std::string def(const TensorType& t, const std::string& expr, bool inBody, bool narrowing = true) {
    const bool strict = strictBf16();
    std::string name = fresh("t");
    const bool inB = inBody || guard_ > 0 || mentionsBody(expr);
    if (inB) bodyNames_.insert(name);
    emit(inB, "const " + computeT(t.dt) + " " + name + " = " + ((strict || narrowing) ? roundTo(t.dt, expr) : expr) + ";");
    return name;
  }

  // guarded evaluation: value = cond ? gen(inner) : other
  template <typename F>
  std::string guarded(const TensorType& t, const std::string& cond, F inner, const std::string& other) {
    std::string name = fresh("t");
    bodyNames_.insert(name);
    body(computeT(t.dt) + " " + name + " = " + other + ";");
    body("if (" + cond + ") {");
    body_.emplace_back();
    cache_.emplace_back();
    ++guard_;
    std::string val = inner();
    --guard_;
    std::string inside = body_.back();
    body_.pop_back();
    cache_.pop_back();
    body_.back() += inside;
    body("  " + name + " = " + val + ";");
    body("}");
    return name;
  }

  std::string genUncached(Value* v, const Index& idx) {
    auto rs = rowScalars_.find(v);
    if (rs != rowScalars_.end()) {
      // only the current row's value exists: the index must be the row index itself
      Index m = multi(idx);
      if (m.dims.size() != rowKept_.size()) throw CompileError("row program: reduction result indexed through a reshape");
      for (size_t q = 0; q < m.dims.size(); ++q) {
        if (v->type.dims[q] == 1) continue;
        const IdxDim& d = m.dims[q];
        if (d.isConst || d.inBody || d.coef != 0 || d.base != rowKept_[q].base) throw CompileError("row program: reduction result read at another row");
      }
      return rs->second;
    }
    if (isLeaf_(v)) return load(v, idx);
    Op* op = v->def;
    if (!op) throw CompileError("codegen: region argument " + v->name + " is not materialised");
    const std::string& n = op->name;
    const TensorType& rt = v->type;
    bool inB = idx.lane();
    auto in = [&](int k) { return gen(op->operands[k], idx); };
    const bool narrowing = n == "convert" || n == "reduce_precision" || n == "bitcast_convert" || n == "iota" || n == "round_nearest_even" ||
                           n == "round_nearest_afz" || n == "floor" || n == "ceil";
    auto bin = [&](const std::string& e) { return def(rt, e, inB, narrowing); };
    DType odt = op->operands.empty() ? rt.dt : op->operands[0]->type.dt;
    bool isF = isFloat(rt.dt), isD = rt.dt == DType::F64, isP = rt.dt == DType::Pred;
    std::string sfx = isD ? "" : "f";

    // ---- structural ops
    if (n == "constant") {
      auto& d = *op->attrs.at("value").dense;
      if (d.splat || d.type.numel() == 1) return literalFromBytes(d.type.dt, d.bytes.data());
      throw CompileError("codegen: dense constant must be materialised");
    }
    if (n == "iota") {
      Index m = multi(idx);
      return def(rt, "(" + computeT(rt.dt) + ")" + dimExpr(m.dims[op->integer("dim")]), inB);
    }
    if (n == "reshape") {
      Value* x = op->operands[0];
      if (idx.linear) return gen(x, linearIndex(idx.lin, x->type.dims));
      // same dims up to unit dims: remap without div/mod
      std::vector<IdxDim> od(x->type.rank());
      size_t a = 0;
      bool simple = true;
      for (int d = 0; d < x->type.rank() && simple; ++d) {
        if (x->type.dims[d] == 1) { od[d] = constDim(0); continue; }
        while (a < rt.dims.size() && rt.dims[a] == 1) ++a;
        if (a < rt.dims.size() && rt.dims[a] == x->type.dims[d]) od[d] = idx.dims[a++];
        else simple = false;
      }
      if (simple) {
        while (a < rt.dims.size() && rt.dims[a] == 1) ++a;
        if (a == rt.dims.size()) return gen(x, multiIndex(od, x->type.dims));
      }
      IdxDim lin = linearize(idx.dims, rt.dims);
      return gen(x, linearIndex(lin, x->type.dims));
    }
    if (n == "broadcast_in_dim") {
      Value* x = op->operands[0];
      auto& dims = op->ints("dims");
      if (x->type.rank() == 0) return gen(x, multiIndex({}, {}));
      Index m = multi(idx);
      std::vector<IdxDim> od(x->type.rank());
      for (int k = 0; k < x->type.rank(); ++k) od[k] = x->type.dims[k] == 1 ? constDim(0) : m.dims[dims[k]];
      return gen(x, multiIndex(od, x->type.dims));
    }
    if (n == "transpose") {
      Value* x = op->operands[0];
      auto& perm = op->ints("dims");
      Index m = multi(idx);
      std::vector<IdxDim> od(x->type.rank());
      for (int k = 0; k < x->type.rank(); ++k) od[perm[k]] = m.dims[k];
      return gen(x, multiIndex(od, x->type.dims));
    }
    if (n == "reverse") {
      Value* x = op->operands[0];
      Index m = multi(idx);
      for (auto d : op->ints("dims")) m.dims[d] = affine(m.dims[d], -1, x->type.dims[d] - 1);
      finishSig(m);
      return gen(x, m);
    }
    if (n == "slice") {
      Value* x = op->operands[0];
      Index m = multi(idx);
      auto& st = op->ints("start");
      auto& sr = op->ints("strides");
      for (int d = 0; d < x->type.rank(); ++d) m.dims[d] = affine(m.dims[d], sr.empty() ? 1 : sr[d], st[d]);
      m.shape = x->type.dims;
      finishSig(m);
      return gen(x, m);
    }
    if (n == "dynamic_slice") {
      Value* x = op->operands[0];
      Index m = multi(idx);
      auto& sizes = op->ints("sizes");
      for (int d = 0; d < x->type.rank(); ++d) {
        int64_t hi = x->type.dims[d] - sizes[d];
        if (hi == 0) continue;   // start is clamped to 0
        std::string s = gen(op->operands[1 + d], multiIndex({}, {}));
        IdxDim st = var("(" + idxT() + ")mn<i64>(mx<i64>((i64)" + s + ", 0), " + std::to_string(hi) + ")", false);
        m.dims[d] = addDims(m.dims[d], st);
      }
      m.shape = x->type.dims;
      finishSig(m);
      return gen(x, m);
    }
    if (n == "pad") {
      Value* x = op->operands[0];
      auto& lo = op->ints("low");
      auto& hi = op->ints("high");
      auto& it = op->ints("interior");
      bool trivial = true;
      for (int d = 0; d < x->type.rank(); ++d) if (lo[d] != 0 || hi[d] != 0 || it[d] != 0) trivial = false;
      if (trivial) return gen(x, idx);
      Index m = multi(idx);
      std::string pv = gen(op->operands[1], multiIndex({}, {}));
      std::string cond;
      std::vector<IdxDim> od(x->type.rank());
      for (int d = 0; d < x->type.rank(); ++d) {
        if (lo[d] == 0 && hi[d] == 0 && it[d] == 0) { od[d] = m.dims[d]; continue; }
        IdxDim s = toBody(affine(m.dims[d], 1, -lo[d]));   // position in the dilated operand
        std::string e = dimExpr(s);
        std::string c = "(" + e + " >= 0)";
        if (it[d] > 0) {
          int64_t q = it[d] + 1;
          c += " && (" + e + " % " + std::to_string(q) + " == 0) && (" + e + " / " + std::to_string(q) + " < " + std::to_string(x->type.dims[d]) + ")";
          IdxDim r;
          r.isConst = false; r.inBody = true; r.base = "(" + e + " / " + std::to_string(q) + ")";
          od[d] = r;
        } else {
          c += " && (" + e + " < " + std::to_string(x->type.dims[d]) + ")";
          od[d] = s;
        }
        cond += (cond.empty() ? "" : " && ") + c;
      }
      Index oi = multiIndex(od, x->type.dims);
      return guarded(rt, cond, [&] { return gen(x, oi); }, pv);
    }
    if (n == "concatenate") {
      int64_t dim = op->integer("dim");
      Index m = multi(idx);
      // lane-invariant along `dim` and not guarded: still emitted in the body for simplicity
      IdxDim pos = toBody(m.dims[dim]);
      std::string e = dimExpr(pos);
      std::string name = fresh("t");
      bodyNames_.insert(name);
      body(computeT(rt.dt) + " " + name + ";");
      int64_t off = 0;
      for (size_t k = 0; k < op->operands.size(); ++k) {
        Value* x = op->operands[k];
        int64_t sz = x->type.dims[dim];
        if (sz == 0) continue;
        bool lastPiece = true;
        for (size_t q = k + 1; q < op->operands.size(); ++q) if (op->operands[q]->type.dims[dim] != 0) lastPiece = false;
        body(std::string(off == 0 ? "if" : "else if") + " (" + (lastPiece ? "true" : e + " < " + std::to_string(off + sz)) + ") {");
        body_.emplace_back();
        cache_.emplace_back();
        ++guard_;
        Index oi = m;
        IdxDim r;
        r.isConst = false; r.inBody = true; r.base = "(" + e + " - " + std::to_string(off) + ")";
        oi.dims[dim] = r;
        oi.shape = x->type.dims;
        finishSig(oi);
        std::string val = gen(x, oi);
        --guard_;
        std::string inside = body_.back();
        body_.pop_back();
        cache_.pop_back();
        body_.back() += inside;
        body("  " + name + " = " + val + ";");
        body("}");
        off += sz;
      }
      return name;
    }
    if (n == "gather") return genGather(op, v, idx);
    if (n == "optimization_barrier") return gen(op->operands[v->defIndex], idx);
    if (n == "custom_call") return in(0);

    // ---- conversions
    if (n == "convert") {
      std::string x = in(0);
      std::string e;
      if (isP) e = "(" + x + " != 0)";
      else if (isFloat(odt) && !isF) e = "f2i<" + computeT(rt.dt) + ", " + computeT(odt) + ">(" + x + ")";
      else e = "(" + computeT(rt.dt) + ")(" + x + ")";
      return bin(e);
    }
    if (n == "bitcast_convert") {
      std::string x = in(0);
      size_t a = dtypeSize(odt), b = dtypeSize(rt.dt);
      if (a != b) throw CompileError("bitcast_convert between element types of different width is not supported");
      auto toBits = [&](DType d, const std::string& e) -> std::string {
        if (d == DType::F32) return "__float_as_uint(" + e + ")";
        if (d == DType::F64) return "(u64)__double_as_longlong(" + e + ")";
        if (d == DType::BF16) return "f2bf(" + e + ")";
        if (d == DType::F16) { return "__half_as_ushort(__float2half(" + e + "))"; }
        return "(" + std::string(b == 1 ? "u8" : b == 2 ? "u16" : b == 4 ? "u32" : "u64") + ")(" + e + ")";
      };
      std::string bits = toBits(odt, x);
      std::string e;
      if (rt.dt == DType::F32) e = "__uint_as_float(" + bits + ")";
      else if (rt.dt == DType::F64) e = "__longlong_as_double((i64)" + bits + ")";
      else if (rt.dt == DType::BF16) e = "bf2f(" + bits + ")";
      else if (rt.dt == DType::F16) e = "__half2float(__ushort_as_half(" + bits + "))";
      else e = "(" + computeT(rt.dt) + ")(" + bits + ")";
      return def(rt, e, inB);
    }
    if (n == "reduce_precision")
      return bin("redprec(" + in(0) + ", " + std::to_string(op->integer("exponent_bits")) + ", " + std::to_string(op->integer("mantissa_bits")) + ")");

    // ---- comparisons / selection
    if (n == "compare") {
      std::string a = in(0), b = in(1);
      const std::string& dir = op->str("direction");
      const char* c = dir == "EQ" ? "==" : dir == "NE" ? "!=" : dir == "LT" ? "<" : dir == "LE" ? "<=" : dir == "GT" ? ">" : ">=";
      if (op->str("compare_type") == "TOTALORDER" && isFloat(odt) && odt != DType::F64) { a = "tokey(" + a + ")"; b = "tokey(" + b + ")"; }
      return bin("(" + a + " " + c + " " + b + ")");
    }
    if (n == "select") {
      Value* p = op->operands[0];
      std::string ps = p->type.rank() == 0 && rt.rank() != 0 ? gen(p, multiIndex({}, {})) : gen(p, idx);
      return bin("(" + ps + " ? " + in(1) + " : " + in(2) + ")");
    }
    if (n == "clamp") {
      auto side = [&](int k) {
        Value* s = op->operands[k];
        return s->type.rank() == 0 && rt.rank() != 0 ? gen(s, multiIndex({}, {})) : gen(s, idx);
      };
      std::string T = computeT(rt.dt);
      return bin("mn<" + T + ">(mx<" + T + ">(" + in(1) + ", " + side(0) + "), " + side(2) + ")");
    }

    // ---- binary arithmetic
    std::string T = computeT(rt.dt);
    const bool wraps = rt.dt == DType::S32 || rt.dt == DType::S64;   // signed overflow has to wrap, not to be assumed away
    if (n == "add") return bin(isP ? "(" + in(0) + " || " + in(1) + ")" : wraps ? "wadd<" + T + ">(" + in(0) + ", " + in(1) + ")" : "(" + in(0) + " + " + in(1) + ")");
    if (n == "subtract") return bin(wraps ? "wsub<" + T + ">(" + in(0) + ", " + in(1) + ")" : "(" + in(0) + " - " + in(1) + ")");
    if (n == "multiply") return bin(isP ? "(" + in(0) + " && " + in(1) + ")" : wraps ? "wmul<" + T + ">(" + in(0) + ", " + in(1) + ")" : "(" + in(0) + " * " + in(1) + ")");
    if (n == "divide") {
      // a divisor that is one number per row (softmax's sum) is inverted once per row, not once per element
      if (isF && !isD) {
        std::string d = in(1);
        auto rc = rowRcp_.find(d);
        if (rc != rowRcp_.end()) return bin("(" + in(0) + " * " + rc->second + ")");
      }
      return bin(isF ? "(" + in(0) + " / " + in(1) + ")" : "idiv<" + T + ">(" + in(0) + ", " + in(1) + ")");
    }
    if (n == "remainder") return bin(isF ? "fmod" + sfx + "(" + in(0) + ", " + in(1) + ")" : "irem<" + T + ">(" + in(0) + ", " + in(1) + ")");
    if (n == "maximum") return bin(isP ? "(" + in(0) + " || " + in(1) + ")" : "mx<" + T + ">(" + in(0) + ", " + in(1) + ")");
    if (n == "minimum") return bin(isP ? "(" + in(0) + " && " + in(1) + ")" : "mn<" + T + ">(" + in(0) + ", " + in(1) + ")");
    if (n == "power") return bin(isF ? "pow" + sfx + "(" + in(0) + ", " + in(1) + ")" : "ipow<" + T + ">(" + in(0) + ", " + in(1) + ")");
    if (n == "atan2") return bin("atan2" + sfx + "(" + in(0) + ", " + in(1) + ")");
    if (n == "and") return bin(isP ? "(" + in(0) + " && " + in(1) + ")" : "(" + T + ")(" + in(0) + " & " + in(1) + ")");
    if (n == "or") return bin(isP ? "(" + in(0) + " || " + in(1) + ")" : "(" + T + ")(" + in(0) + " | " + in(1) + ")");
    if (n == "xor") return bin(isP ? "(" + in(0) + " != " + in(1) + ")" : "(" + T + ")(" + in(0) + " ^ " + in(1) + ")");
    if (n == "shift_left" || n == "shift_right_logical" || n == "shift_right_arithmetic") {
      int bits = (int)dtypeSize(rt.dt) * 8;
      std::string U = bits == 8 ? "u8" : bits == 16 ? "u16" : bits == 32 ? "u32" : "u64";
      std::string a = in(0), s = in(1);
      std::string inr = "((u64)(" + s + ") < " + std::to_string(bits) + "ull)";
      if (n == "shift_left") return bin("(" + inr + " ? (" + T + ")((" + U + ")" + a + " << (" + s + ")) : (" + T + ")0)");
      if (n == "shift_right_logical") return bin("(" + inr + " ? (" + T + ")((" + U + ")" + a + " >> (" + s + ")) : (" + T + ")0)");
      return bin("(" + T + ")(" + a + " >> (" + inr + " ? (int)(" + s + ") : " + std::to_string(bits - 1) + "))");
    }

    // ---- unary
    if (n == "negate") return bin(isP ? in(0) : wraps ? "wsub<" + T + ">((" + T + ")0, " + in(0) + ")" : "(" + T + ")(-" + in(0) + ")");
    if (n == "abs") return bin(isF ? "fabs" + sfx + "(" + in(0) + ")" : wraps ? "(" + in(0) + " < 0 ? wsub<" + T + ">((" + T + ")0, " + in(0) + ") : " + in(0) + ")" : "(" + T + ")(" + in(0) + " < 0 ? -" + in(0) + " : " + in(0) + ")");
    if (n == "not") return bin(isP ? "(!" + in(0) + ")" : "(" + T + ")(~" + in(0) + ")");
    if (n == "sign") return bin(isF ? (isD ? "sgnd(" : "sgnf(") + in(0) + ")" : "(" + T + ")((" + in(0) + " > 0) - (" + in(0) + " < 0))");
    if (n == "is_finite") return bin("isfinite(" + in(0) + ")");
    const bool half = rt.dt == DType::BF16 || rt.dt == DType::F16;
    if (half && n == "tanh") {
      // read only by an addition of a constant of magnitude 1/2 or more: the sum hides what the difference of exponentials
      // loses near zero (6e-8 absolute)
      bool absorbed = v->users.size() == 1 && v->users[0]->name == "add" && v->users[0]->operands.size() == 2;
      if (absorbed) {
        Op* u = v->users[0];
        Value* other = u->operands[0] == v ? u->operands[1] : u->operands[0];
        Op* d = other->def;
        while (d && (d->name == "broadcast_in_dim" || d->name == "reshape" || d->name == "convert") && d->operands.size() == 1) d = d->operands[0]->def;
        absorbed = false;
        if (other != v && d && d->name == "constant" && d->has("value") && d->attrs.at("value").dense) {
          const DenseData& dd = *d->attrs.at("value").dense;
          if ((dd.splat || dd.type.numel() == 1) && isFloat(dd.type.dt)) {
            const std::string lit = literalFromBytes(dd.type.dt, dd.bytes.data());   // "__uint_as_float(0x...u)" for the 32- and 16-bit types
            const size_t at = lit.find("0x");
            if (dd.type.dt != DType::F64 && at != std::string::npos) {
              const uint32_t bits = (uint32_t)strtoul(lit.c_str() + at, nullptr, 16);
              float c;
              memcpy(&c, &bits, 4);
              absorbed = std::fabs(c) >= 0.5f && std::isfinite(c);
            }
          }
        }
      }
      return bin(std::string(absorbed ? "tanh_fast_abs(" : "tanh_fast(") + in(0) + ")");
    }
    if (half && n == "exponential") return bin("__expf(" + in(0) + ")");
    if (rt.dt == DType::F32 && n == "tanh") return bin("tanh_f32(" + in(0) + ")");
    if (half && n == "logistic") return bin("(1.f / (1.f + __expf(-" + in(0) + ")))");
    if (n == "logistic") return bin(isD ? "(1.0 / (1.0 + exp(-" + in(0) + ")))" : "(1.f / (1.f + expf(-" + in(0) + ")))");
    if (n == "rsqrt") return bin(isD ? "(1.0 / sqrt(" + in(0) + "))" : "(1.f / sqrtf(" + in(0) + "))");
    if (n == "popcnt") return bin(dtypeSize(rt.dt) == 8 ? "(" + T + ")__popcll((u64)" + in(0) + ")" : "(" + T + ")__popc((u32)(" + std::string(dtypeSize(rt.dt) == 4 ? "u32" : dtypeSize(rt.dt) == 2 ? "u16" : "u8") + ")" + in(0) + ")");
    if (n == "count_leading_zeros") {
      int bits = (int)dtypeSize(rt.dt) * 8;
      if (bits == 64) return bin("(" + T + ")__clzll((i64)" + in(0) + ")");
      std::string U = bits == 8 ? "u8" : bits == 16 ? "u16" : "u32";
      return bin("(" + T + ")(__clz((int)(u32)(" + U + ")" + in(0) + ") - " + std::to_string(32 - bits) + ")");
    }
    if (n == "round_nearest_afz" && isF) {
      // the reference's formula, sign(x) * floor(|x| + 0.5) in the operand type (ops/arithmetic.cc:316-327): where the sum
      // is not representable it rounds first, so the predecessor of 0.5 gives 1 and an odd integer from 2^23 on (2^7 for
      // bf16, 2^10 for f16) its even neighbour; an exact rounding would differ from the reference there
      const std::string x = in(0);
      const std::string sum = roundTo(rt.dt, "(fabs" + sfx + "(" + x + ") + " + (isD ? "0.5" : "0.5f") + ")");
      const std::string FT = isD ? "double" : "float";   // (the sign as the difference of two comparisons: zero for either zero)
      return bin("((" + FT + ")((" + x + " > 0) - (" + x + " < 0)) * floor" + sfx + "(" + sum + "))");
    }
    static const std::unordered_map<std::string, const char*> unary = {
        {"exponential", "exp"}, {"exponential_minus_one", "expm1"}, {"log", "log"}, {"log_plus_one", "log1p"},
        {"sqrt", "sqrt"}, {"cbrt", "cbrt"}, {"tanh", "tanh"}, {"tan", "tan"}, {"sine", "sin"}, {"cosine", "cos"},
        {"floor", "floor"}, {"ceil", "ceil"}, {"round_nearest_even", "rint"}, {"round_nearest_afz", "round"},
        // chlo unary ops, also reached as custom_call @mhlo.<name> (reference: ops/control_flow.cc:53-63)
        {"chlo.asin", "asin"}, {"chlo.acos", "acos"}, {"chlo.atan", "atan"}, {"chlo.sinh", "sinh"}, {"chlo.cosh", "cosh"},
        {"chlo.asinh", "asinh"}, {"chlo.acosh", "acosh"}, {"chlo.atanh", "atanh"}, {"chlo.erf", "erf"},
        {"chlo.erf_inv", "erfinv"}};
    auto it = unary.find(n);
    if (it != unary.end()) return bin(std::string(it->second) + sfx + "(" + in(0) + ")");
    throw CompileError("codegen: no lowering for stablehlo." + n);
  }

  // stablehlo.gather as index arithmetic: every start index is clamped into
  // [0, dim - slice] (reference: ops/gather_scatter.cc:233-239).
  std::string genGather(Op* op, Value* v, const Index& idx) {
    Value* operand = op->operands[0];
    Value* indices = op->operands[1];
    auto& offsetDims = op->ints("offset_dims");
    auto& collapsed = op->ints("collapsed_slice_dims");
    auto& obatch = op->ints("operand_batching_dims");
    auto& ibatch = op->ints("start_indices_batching_dims");
    auto& sim = op->ints("start_index_map");
    int64_t ivd = op->integer("index_vector_dim");
    auto& sizes = op->ints("slice_sizes");
    auto has = [](const std::vector<int64_t>& a, int64_t x) { return std::find(a.begin(), a.end(), x) != a.end(); };
    Index m = multi(idx);
    int rank = v->type.rank();
    std::vector<IdxDim> batchIdx, offIdx;
    for (int d = 0; d < rank; ++d) (has(offsetDims, d) ? offIdx : batchIdx).push_back(m.dims[d]);
    int irank = indices->type.rank();
    auto indexAt = [&](int k) {
      std::vector<IdxDim> id(irank);
      size_t b = 0;
      for (int d = 0; d < irank; ++d) {
        if (d == ivd) id[d] = constDim(k);
        else id[d] = batchIdx.at(b++);
      }
      return multiIndex(id, indices->type.dims);
    };
    int orank = operand->type.rank();
    std::vector<IdxDim> od(orank, constDim(0));
    for (size_t k = 0; k < sim.size(); ++k) {
      int64_t d = sim[k];
      int64_t hi = operand->type.dims[d] - sizes[d];
      if (hi <= 0) continue;
      Index ii = indexAt((int)k);
      std::string s = gen(indices, ii);
      IdxDim st = var("(" + idxT() + ")mn<i64>(mx<i64>((i64)" + s + ", 0), " + std::to_string(hi) + ")", ii.lane());
      od[d] = st;
    }
    // batching dims take the coordinate of the matching batch dim of the indices
    std::vector<int> idxBatchAxes;
    for (int d = 0; d < irank; ++d) if (d != ivd) idxBatchAxes.push_back(d);
    for (size_t k = 0; k < obatch.size(); ++k) {
      int pos = (int)(std::find(idxBatchAxes.begin(), idxBatchAxes.end(), (int)ibatch[k]) - idxBatchAxes.begin());
      od[obatch[k]] = addDims(od[obatch[k]], batchIdx.at(pos));
    }
    size_t o = 0;
    for (int d = 0; d < orank; ++d) {
      if (has(collapsed, d) || has(obatch, d)) continue;
      od[d] = addDims(od[d], offIdx.at(o++));
    }
    return gen(operand, multiIndex(od, operand->type.dims));
  }
};

int pickVector(const TensorType& t) {
  int v = (int)std::max<size_t>(1, 16 / std::max<size_t>(1, dtypeSize(t.dt)));
  v = std::min(v, 8);
  int64_t last = t.rank() ? t.dims.back() : 1;
  // the innermost dim of size 1 carries no information: use the product of trailing dims instead
  int64_t n = t.numel();
  int64_t trail = last;
  for (int d = t.rank() - 2; d >= 0 && trail == 1; --d) trail = t.dims[d];
  (void)n;
  while (v > 1 && trail % v != 0) v >>= 1;
  return v;
}

bool needs64(const std::vector<Value*>& vals) {
  for (auto* v : vals) if (v->type.numel() >= (int64_t(1) << 31) - 16) return true;
  return false;
}

std::string kernelHeader(const std::vector<Value*>& leaves, const std::vector<std::string>& outs) {
  std::string s = "extern \"C\" __global__ void __launch_bounds__(256) k(";
  bool first = true;
  for (size_t i = 0; i < leaves.size(); ++i) {
    s += std::string(first ? "" : ", ") + "const " + storageT(leaves[i]->type.dt) + "* __restrict__ in" + std::to_string(i);
    first = false;
  }
  for (auto& o : outs) {
    s += std::string(first ? "" : ", ") + o;
    first = false;
  }
  return s + ")";
}

void collectAllValues(Value* root, const LeafPredicate& isLeaf, std::vector<Value*>& out, std::unordered_map<Value*, bool>& seen) {
  if (seen[root]) return;
  seen[root] = true;
  out.push_back(root);
  if (isLeaf(root) || !root->def) return;
  for (auto* o : root->def->operands) collectAllValues(o, isLeaf, out, seen);
}

}  // namespace

bool isFusibleOp(const Op& op) {
  static const char* names[] = {
      "add", "subtract", "multiply", "divide", "maximum", "minimum", "power", "remainder", "atan2", "and", "or", "xor",
      "not", "negate", "abs", "exponential", "exponential_minus_one", "log", "log_plus_one", "sqrt", "rsqrt", "cbrt",
      "tanh", "tan", "sine", "cosine", "logistic", "floor", "ceil", "sign", "round_nearest_even", "round_nearest_afz",
      "is_finite", "shift_left", "shift_right_logical", "shift_right_arithmetic", "popcnt", "count_leading_zeros",
      "compare", "select", "clamp", "convert", "bitcast_convert", "reduce_precision", "constant", "iota", "reshape",
      "broadcast_in_dim", "transpose", "reverse", "concatenate", "slice", "dynamic_slice", "pad", "gather",
      "optimization_barrier", "custom_call", "chlo.asin", "chlo.acos", "chlo.atan", "chlo.sinh", "chlo.cosh", "chlo.asinh",
      "chlo.acosh", "chlo.atanh", "chlo.erf", "chlo.erf_inv"};
  for (auto* n : names) if (op.name == n) return true;
  return false;
}

static const char* reduceKind(const Op& reduce) {
  if (reduce.regions.size() != 1) return nullptr;
  auto& r = *reduce.regions[0];
  if (r.args.size() != 2 || r.ops.size() != 2) return nullptr;
  Op* b = r.ops[0].get();
  Op* ret = r.ops[1].get();
  if (ret->name != "return" || ret->operands.size() != 1 || ret->operands[0] != b->result()) return nullptr;
  if (b->operands.size() != 2) return nullptr;
  bool uses = (b->operands[0] == r.args[0].get() && b->operands[1] == r.args[1].get()) ||
              (b->operands[0] == r.args[1].get() && b->operands[1] == r.args[0].get());
  if (!uses) return nullptr;
  for (const char* k : {"add", "multiply", "maximum", "minimum", "and", "or"})
    if (b->name == k) return k;
  return nullptr;
}

bool isSimpleReduce(const Op& reduce) { return reduce.operands.size() == 2 && reduceKind(reduce) != nullptr; }
const char* simpleReduceKind(const Op& reduce) { return reduce.operands.size() == 2 ? reduceKind(reduce) : nullptr; }

// ------------------------------------------------------------------ loop kernels
static constexpr int64_t kSpreadThreads = 65536;   // lanes a small kernel is spread over before its lanes take vectors (256 compute units x 256)

FusedCode generateLoopKernel(Value* root, const LeafPredicate& isLeaf) { return generateLoopKernel(std::vector<Value*>{root}, isLeaf); }

// One pass over a shared index space that stores several results: all roots have the same
// dims; a root may feed another root (it is then computed once and both are stored).
FusedCode generateLoopKernel(const std::vector<Value*>& roots, const LeafPredicate& isLeaf) {
  std::vector<Value*> all;
  std::unordered_map<Value*, bool> seen;
  auto isRoot = [&](Value* v) { return std::find(roots.begin(), roots.end(), v) != roots.end(); };
  LeafPredicate inner = [&](Value* v) { return !isRoot(v) && isLeaf(v); };
  for (auto* r : roots) collectAllValues(r, inner, all, seen);
  Value* root = roots[0];
  int V = 8;
  for (auto* r : roots) V = std::min(V, pickVector(r->type));
  bool i64 = needs64(all);
  int64_t N = root->type.numel();
  // a small index space is spread over more lanes instead of vectors: a lane that walks four elements of a chain of
  // exponentials in turn takes four times as long, and nothing this size is bound by memory transactions
  while (V > 1 && N / V < kSpreadThreads) V >>= 1;
  Emitter em(inner, V, i64);
  IdxDim lin;
  lin.isConst = false;
  lin.base = "base";
  lin.coef = 1;
  lin.mult = V;
  if (V == 1) { lin.coef = 0; }
  Index idx = em.linearIndex(lin, root->type.dims);
  std::vector<std::string> vals;
  for (auto* r : roots) vals.push_back(em.gen(r, idx));
  std::ostringstream s;
  s << kPrelude;
  std::vector<std::string> outs;
  for (size_t j = 0; j < roots.size(); ++j) outs.push_back(storageT(roots[j]->type.dt) + "* __restrict__ out" + std::to_string(j));
  s << kernelHeader(em.leaves_, outs) << " {\n";
  s << "  const " << em.idxT() << " base = ((" << em.idxT() << ")blockIdx.x * 256 + threadIdx.x) * " << V << ";\n";
  s << "  if (base >= " << N << (i64 ? "ll" : "") << ") return;\n";
  s << em.pre_;
  if (V > 1) {
    for (size_t j = 0; j < roots.size(); ++j) s << "  Vec<" << storageT(roots[j]->type.dt) << ", " << V << "> ov" << j << ";\n";
    s << "  #pragma unroll\n  for (int v = 0; v < " << V << "; ++v) {\n";
    s << em.body_.front();
    for (size_t j = 0; j < roots.size(); ++j) s << "    ov" << j << ".e[v] = " << storeExpr(roots[j]->type.dt, vals[j]) << ";\n";
    s << "  }\n";
    for (size_t j = 0; j < roots.size(); ++j)
      s << "  *(Vec<" << storageT(roots[j]->type.dt) << ", " << V << ">*)(out" << j << " + base) = ov" << j << ";\n";
  } else {
    s << "  {\n    const int v = 0; (void)v;\n" << em.body_.front();
    for (size_t j = 0; j < roots.size(); ++j) s << "    out" << j << "[base] = " << storeExpr(roots[j]->type.dt, vals[j]) << ";\n";
    s << "  }\n";
  }
  s << "}\n";
  FusedCode fc;
  Launch l;
  l.source = s.str();
  int64_t threads = (N + V - 1) / V;
  l.grid[0] = (unsigned)std::max<int64_t>(1, (threads + 255) / 256);
  l.block[0] = 256;
  for (auto* v : em.leaves_) { KArg a; a.kind = KArg::In; a.value = v; l.args.push_back(a); }
  for (auto* r : roots) {
    KArg o;
    o.kind = KArg::Out;
    o.value = r;
    l.args.push_back(o);
  }
  fc.launches.push_back(std::move(l));
  fc.leaves = em.leaves_;
  return fc;
}

// -------------------------------------------------- dynamic_update_slice window
FusedCode generateDusKernel(Op* dus, const LeafPredicate& isLeaf) {
  Value* operand = dus->operands[0];
  Value* update = dus->operands[1];
  Value* result = dus->result();
  std::vector<Value*> all;
  std::unordered_map<Value*, bool> seen;
  collectAllValues(update, isLeaf, all, seen);
  for (size_t k = 2; k < dus->operands.size(); ++k) collectAllValues(dus->operands[k], isLeaf, all, seen);
  all.push_back(operand);
  int V = pickVector(update->type);
  // the window start along the innermost dim is data dependent, so stores are per lane
  bool i64 = needs64(all);
  Emitter em(isLeaf, V, i64);
  int64_t N = update->type.numel();
  IdxDim lin;
  lin.isConst = false;
  lin.base = "base";
  lin.coef = V > 1 ? 1 : 0;
  lin.mult = V;
  Index idx = em.linearIndex(lin, update->type.dims);
  std::string val = em.gen(update, idx);
  Index m = em.multi(idx);
  std::vector<IdxDim> od(operand->type.rank());
  for (int d = 0; d < operand->type.rank(); ++d) {
    int64_t hi = operand->type.dims[d] - update->type.dims[d];
    if (hi <= 0) { od[d] = m.dims[d]; continue; }
    std::string sidx = em.gen(dus->operands[2 + d], em.multiIndex({}, {}));
    IdxDim st = em.var("(" + em.idxT() + ")mn<i64>(mx<i64>((i64)" + sidx + ", 0), " + std::to_string(hi) + ")", false);
    od[d] = em.addDims(m.dims[d], st);
  }
  IdxDim off = em.linearize(od, operand->type.dims);
  DType dt = result->type.dt;
  std::ostringstream s;
  s << kPrelude;
  s << kernelHeader(em.leaves_, {storageT(dt) + "* out0"}) << " {\n";
  s << "  const " << em.idxT() << " base = ((" << em.idxT() << ")blockIdx.x * 256 + threadIdx.x) * " << V << ";\n";
  s << "  if (base >= " << N << (i64 ? "ll" : "") << ") return;\n";
  s << em.pre_;
  s << "  #pragma unroll\n  for (int v = 0; v < " << V << "; ++v) {\n";
  s << em.body_.front();
  s << "    out0[" << em.dimExpr(off) << "] = " << storeExpr(dt, val) << ";\n  }\n}\n";
  FusedCode fc;
  Launch l;
  l.source = s.str();
  int64_t threads = (N + V - 1) / V;
  l.grid[0] = (unsigned)std::max<int64_t>(1, (threads + 255) / 256);
  l.block[0] = 256;
  for (auto* v : em.leaves_) { KArg a; a.kind = KArg::In; a.value = v; l.args.push_back(a); }
  KArg o;
  o.kind = KArg::Out;
  o.value = result;
  l.args.push_back(o);
  fc.launches.push_back(std::move(l));
  fc.leaves = em.leaves_;
  return fc;
}

// --------------------------------------------------------------- reductions
namespace {

struct RedOp {
  const char* kind;
  DType dt;       // element type of the reduce result
  std::string accT;
  std::string identity;
  // Boolean forms use the non-short-circuit operators: the second operand may be a
  // wavefront shuffle that every lane has to execute.
  std::string combine(const std::string& a, const std::string& b) const {
    std::string k = kind;
    bool p = dt == DType::Pred;
    std::string band = "(bool)((int)" + a + " & (int)" + b + ")", bor = "(bool)((int)" + a + " | (int)" + b + ")";
    const bool wraps = dt == DType::S32 || dt == DType::S64;
    if (k == "add") return p ? bor : wraps ? "wadd<" + accT + ">(" + a + ", " + b + ")" : "(" + a + " + " + b + ")";
    if (k == "multiply") return p ? band : wraps ? "wmul<" + accT + ">(" + a + ", " + b + ")" : "(" + a + " * " + b + ")";
    if (k == "maximum") return p ? bor : "mx<" + accT + ">(" + a + ", " + b + ")";
    if (k == "minimum") return p ? band : "mn<" + accT + ">(" + a + ", " + b + ")";
    if (k == "and") return p ? band : "(" + accT + ")(" + a + " & " + b + ")";
    return p ? bor : "(" + accT + ")(" + a + " | " + b + ")";
  }
};

RedOp makeRedOp(const Op& reduce) {
  RedOp r;
  r.kind = reduceKind(reduce);
  r.dt = reduce.result()->type.dt;
  r.accT = computeT(r.dt);
  std::string k = r.kind;
  bool f = isFloat(r.dt);
  if (k == "add" || k == "or") r.identity = r.dt == DType::Pred ? "false" : "(" + r.accT + ")0";
  else if (k == "multiply") r.identity = r.dt == DType::Pred ? "true" : "(" + r.accT + ")1";
  else if (k == "and") r.identity = r.dt == DType::Pred ? "true" : "(" + r.accT + ")~(" + r.accT + ")0";
  else if (k == "maximum") {
    if (f) r.identity = r.dt == DType::F64 ? "(-__builtin_inf())" : "(-__builtin_inff())";
    else if (r.dt == DType::Pred) r.identity = "false";
    else if (isUnsigned(r.dt)) r.identity = "(" + r.accT + ")0";
    else r.identity = "(" + r.accT + ")(1ull << " + std::to_string(dtypeSize(r.dt) * 8 - 1) + ")";
  } else {
    if (f) r.identity = r.dt == DType::F64 ? "__builtin_inf()" : "__builtin_inff()";
    else if (r.dt == DType::Pred) r.identity = "true";
    else if (isUnsigned(r.dt)) r.identity = "(" + r.accT + ")~(" + r.accT + ")0";
    else r.identity = "(" + r.accT + ")((1ull << " + std::to_string(dtypeSize(r.dt) * 8 - 1) + ") - 1ull)";
  }
  return r;
}

// shuffle of an accumulator across the wavefront (64 lanes), by type width
std::string shflXor(const std::string& accT, const std::string& x, const std::string& lanes) {
  if (accT == "bool") return "(__shfl_xor((int)" + x + ", " + lanes + ", 64) != 0)";
  if (accT == "i8" || accT == "u8" || accT == "i16" || accT == "u16") return "(" + accT + ")__shfl_xor((int)" + x + ", " + lanes + ", 64)";
  return "__shfl_xor(" + x + ", " + lanes + ", 64)";
}

}  // namespace

int64_t reduceOnePassLimit() {
  static const int64_t limit = getenv("MI355X_REDUCE_ONE_PASS") ? atoll(getenv("MI355X_REDUCE_ONE_PASS")) : 256 * 1024;
  return limit;
}

bool reduceIsColumnStyle(const Op* reduce) {
  const std::vector<int64_t>& shape = reduce->operands[0]->type.dims;
  const int rank = (int)shape.size();
  if (rank == 0) return false;
  std::vector<bool> isRed(rank, false);
  for (auto d : reduce->ints("dimensions")) if (d >= 0 && d < rank) isRed[(size_t)d] = true;
  int64_t Kn = 1;
  for (int d = 0; d < rank; ++d) if (!isRed[d]) Kn *= shape[d];
  int inner = rank - 1;
  while (inner > 0 && shape[inner] == 1) --inner;
  return !isRed[inner] && Kn != 1;   // the same rule as in generateReduceKernel
}

FusedCode generateReduceKernel(const std::vector<Op*>& reduces, const LeafPredicate& isLeafOuter, const std::vector<Value*>& epilogue, int64_t externalPartials,
                               const std::vector<Value*>& sideStores) {
  // values computed from the results right where they are finished (second pass only)
  std::unordered_set<Value*> own;
  for (auto* r : reduces) own.insert(r->result());
  for (auto* v : epilogue) own.insert(v);
  LeafPredicate isLeaf = [&](Value* v) { return !own.count(v) && isLeafOuter(v); };
  Op* r0 = reduces[0];
  Value* x0 = r0->operands[0];
  const std::vector<int64_t>& shape = x0->type.dims;
  int rank = (int)shape.size();
  std::vector<int64_t> rdims = r0->ints("dimensions");
  std::sort(rdims.begin(), rdims.end());
  std::vector<bool> isRed(rank, false);
  for (auto d : rdims) isRed[d] = true;
  std::vector<int64_t> keptShape, redShape;
  std::vector<int> keptDims, redDims;
  for (int d = 0; d < rank; ++d) {
    if (isRed[d]) { redShape.push_back(shape[d]); redDims.push_back(d); }
    else { keptShape.push_back(shape[d]); keptDims.push_back(d); }
  }
  int64_t Kn = 1, Rn = 1;
  for (auto d : keptShape) Kn *= d;
  for (auto d : redShape) Rn *= d;
  size_t nr = reduces.size();
  std::vector<RedOp> ops;
  for (auto* r : reduces) ops.push_back(makeRedOp(*r));

  std::vector<Value*> all;
  std::unordered_map<Value*, bool> seen;
  for (auto* r : reduces) {
    collectAllValues(r->operands[0], isLeaf, all, seen);
    collectAllValues(r->operands[1], isLeaf, all, seen);
  }
  bool i64 = needs64(all);
  std::string IT = i64 ? "i64" : "int";

  // innermost non-unit dim decides the strategy
  int inner = rank - 1;
  while (inner > 0 && shape[inner] == 1) --inner;
  bool rowStyle = rank == 0 || isRed[inner] || Kn == 1;
  FusedCode fc;

  // ---- common: the final pass that folds partials and the init value
  auto finalPass = [&](int64_t P, int64_t workStride, std::vector<int64_t> workOff, std::vector<Value*>& initLeaves) -> Launch {
    // out[k] = combine(init, partial[0..P)[k])
    Emitter em(isLeaf, 1, i64);
    std::vector<std::string> inits;
    for (auto* r : reduces) inits.push_back(em.gen(r->operands[1], em.multiIndex({}, {})));
    std::ostringstream s;   // body; the header follows once the epilogue has named its inputs
    std::vector<std::string> outs;
    for (size_t j = 0; j < nr; ++j) outs.push_back("const " + ops[j].accT + "* __restrict__ part" + std::to_string(j));
    for (size_t j = 0; j < nr; ++j) outs.push_back(storageT(ops[j].dt) + "* __restrict__ out" + std::to_string(j));
    for (size_t q = 0; q < epilogue.size(); ++q) outs.push_back(storageT(epilogue[q]->type.dt) + "* __restrict__ outE" + std::to_string(q));
    // many partials per output: one wavefront folds an output (lanes stride over the
    // partials, then a butterfly); few partials: one lane per output
    // a whole workgroup per output when there are hundreds of partials (every lane issues its few
    // loads at once, so the fold costs one memory round trip)
    const bool blockPerOut = P >= 256;
    const bool wavePerOut = !blockPerOut && P >= 16;
    if (blockPerOut) {
      s << "  const int lane = threadIdx.x & 63;\n";
      s << "  const " << IT << " kk = (" << IT << ")blockIdx.x;\n";
    } else if (wavePerOut) {
      s << "  const int lane = threadIdx.x & 63;\n";
      s << "  const " << IT << " kk = (" << IT << ")blockIdx.x * 4 + (threadIdx.x >> 6);\n  if (kk >= " << Kn << ") return;\n";
    } else {
      s << "  const " << IT << " kk = (" << IT << ")blockIdx.x * 256 + threadIdx.x;\n  if (kk >= " << Kn << ") return;\n";
    }
    const std::string initPre = em.pre_;
    s << initPre;
    for (size_t j = 0; j < nr; ++j) {
      // partial p of output kk lives at [kk * P + p]: the lanes that fold one output read consecutive words (with the
      // partials of one pass side by side instead, each lane of the fold touched a cache line of its own)
      std::string part = "part" + std::to_string(j) + "[kk * " + std::to_string(P) + " + p]";
      std::string ST = ops[j].accT == "bool" ? "int" : ops[j].accT;
      std::string a = "a" + std::to_string(j);
      s << "  " << ops[j].accT << " " << a << " = " << ops[j].identity << ";\n";
      if (blockPerOut) {
        s << "  #pragma unroll 8\n  for (" << IT << " p = threadIdx.x; p < " << P << "; p += 256) " << a << " = " << ops[j].combine(a, part) << ";\n";
        s << "  #pragma unroll\n  for (int o = 32; o > 0; o >>= 1) " << a << " = " << ops[j].combine(a, shflXor(ops[j].accT, a, "o")) << ";\n";
        s << "  __shared__ " << ST << " fm" << j << "[4];\n";
        s << "  if (lane == 0) fm" << j << "[threadIdx.x >> 6] = " << a << ";\n";
      } else if (wavePerOut) {
        s << "  #pragma unroll 4\n  for (" << IT << " p = lane; p < " << P << "; p += 64) " << a << " = " << ops[j].combine(a, part) << ";\n";
        s << "  #pragma unroll\n  for (int o = 32; o > 0; o >>= 1) " << a << " = " << ops[j].combine(a, shflXor(ops[j].accT, a, "o")) << ";\n";
      } else {
        s << "  for (" << IT << " p = 0; p < " << P << "; ++p) " << a << " = " << ops[j].combine(a, part) << ";\n";
      }
    }
    if (blockPerOut) s << "  __syncthreads();\n  if (threadIdx.x != 0) return;\n";
    else if (wavePerOut) s << "  if (lane != 0) return;\n";
    for (size_t j = 0; j < nr; ++j) {
      std::string a = "a" + std::to_string(j);
      if (blockPerOut) {
        s << "  " << a << " = (" << ops[j].accT << ")fm" << j << "[0];\n";
        s << "  for (int w = 1; w < 4; ++w) " << a << " = " << ops[j].combine(a, "(" + ops[j].accT + ")fm" + std::to_string(j) + "[w]") << ";\n";
      }
      s << "  const " << ops[j].accT << " res" << j << " = " << roundTo(ops[j].dt, ops[j].combine(inits[j], a)) << ";\n";
      s << "  out" << j << "[kk] = " << storeExpr(ops[j].dt, "res" + std::to_string(j)) << ";\n";
    }
    if (!epilogue.empty()) {
      // per-output values that only need the finished results: computed by the lane that holds them
      for (size_t j = 0; j < nr; ++j) em.rowScalars_[reduces[j]->result()] = "res" + std::to_string(j);
      IdxDim klin;
      klin.isConst = false; klin.base = "kk"; klin.coef = 0; klin.mult = 1;
      em.pre_.clear();
      const size_t bodyMark = em.body_.front().size();
      auto kd = em.delinearize(klin, keptShape);
      em.rowKept_ = kd;
      Index kidx = em.multiIndex(kd, keptShape);
      std::vector<std::string> ev;
      for (auto* v : epilogue) ev.push_back(em.gen(v, kidx));
      // (guarded reads, of a padded or concatenated operand say, are written as body statements whatever their index)
      s << em.pre_ << "  { const int v = 0; (void)v;\n" << em.body_.front().substr(bodyMark);
      for (size_t q = 0; q < epilogue.size(); ++q) s << "  outE" << q << "[kk] = " << storeExpr(epilogue[q]->type.dt, ev[q]) << ";\n";
      s << "  }\n";
    }
    s << "}\n";
    Launch l;
    l.source = std::string(kPrelude) + kernelHeader(em.leaves_, outs) + " {\n" + s.str();
    l.grid[0] = (unsigned)(blockPerOut ? Kn : wavePerOut ? (Kn + 3) / 4 : (Kn + 255) / 256);
    l.block[0] = 256;
    for (auto* v : em.leaves_) { KArg a; a.kind = KArg::In; a.value = v; l.args.push_back(a); }
    for (size_t j = 0; j < nr; ++j) { KArg a; a.kind = KArg::Work; a.workOffset = workOff[j]; l.args.push_back(a); }
    for (size_t j = 0; j < nr; ++j) { KArg a; a.kind = KArg::Out; a.value = reduces[j]->result(); l.args.push_back(a); }
    for (auto* v : epilogue) { KArg a; a.kind = KArg::Out; a.value = v; l.args.push_back(a); }
    initLeaves = em.leaves_;
    (void)workStride;
    return l;
  };

  if (externalPartials > 0) {
    std::vector<int64_t> workOff;
    int64_t wb = 0;
    for (size_t j = 0; j < nr; ++j) {
      workOff.push_back(wb);
      wb += (externalPartials * Kn * 8 + 255) / 256 * 256;
    }
    std::vector<Value*> il;
    fc.launches.push_back(finalPass(externalPartials, Kn, workOff, il));
    fc.epilogueFused = !epilogue.empty();
    fc.leaves = il;
    fc.workspaceBytes = wb;
    fc.partialOffsets = workOff;
    return fc;
  }
  if (rowStyle) {
    // lanes run along the reduced elements (r, row-major over the reduced dims).  One
    // wavefront per output when rows are short, one workgroup per output when they
    // are long, and several workgroups per output (partials) when outputs are few.
    int V = 1;
    {
      int64_t lastRed = redShape.empty() ? 1 : redShape.back();
      int v = (int)std::min<size_t>(8, std::max<size_t>(1, 16 / std::max<size_t>(1, dtypeSize(x0->type.dt))));
      bool innerIsLastRed = !redDims.empty() && redDims.back() == inner;
      while (v > 1 && (!innerIsLastRed || lastRed % v != 0)) v >>= 1;
      if (Rn < 64 * v) v = 1;
      V = v;
    }
    int64_t vecs = (Rn + V - 1) / V;
    bool wavePerRow = vecs <= 256 && Kn >= 4;
    int64_t P = 1;                 // workgroups per output row
    static const int perThread = getenv("MI355X_REDUCE_PER_THREAD") ? atoi(getenv("MI355X_REDUCE_PER_THREAD")) : 8;
    static const int rowUnroll = getenv("MI355X_REDUCE_UNROLL") ? atoi(getenv("MI355X_REDUCE_UNROLL")) : 4;
    if (!wavePerRow && Kn < 512 && vecs > 256 * 16) {
      P = std::min<int64_t>((vecs + 256 * perThread - 1) / (256 * perThread), std::max<int64_t>(1, 8192 / Kn));
    }
    Emitter em(isLeaf, V, i64);
    // kept index: lane-invariant
    IdxDim klin;
    klin.isConst = false; klin.base = "kk"; klin.coef = 0; klin.mult = 1;
    auto kd = em.delinearize(klin, keptShape);
    IdxDim rlin;
    rlin.isConst = false; rlin.base = "rb"; rlin.coef = V > 1 ? 1 : 0; rlin.mult = V;
    // everything that depends on rb belongs to the loop body: emit index math there
    std::string savedPre = em.pre_;
    em.pre_.clear();
    auto rd = em.delinearize(rlin, redShape);
    std::vector<IdxDim> full(rank);
    for (size_t q = 0; q < keptDims.size(); ++q) full[keptDims[q]] = kd[q];
    for (size_t q = 0; q < redDims.size(); ++q) full[redDims[q]] = rd[q];
    Index idx = em.multiIndex(full, shape);
    std::vector<std::string> vals;
    for (auto* r : reduces) vals.push_back(em.gen(r->operands[0], idx));
    std::string loopPre = em.pre_;   // statements that depend on rb (per iteration, lane-invariant)
    em.pre_ = savedPre;
    std::vector<std::string> inits;
    for (auto* r : reduces) inits.push_back(em.gen(r->operands[1], em.multiIndex({}, {})));

    std::ostringstream s;   // body; the header follows once an epilogue has named its inputs
    std::vector<std::string> outs;
    bool partial = P > 1;
    for (size_t j = 0; j < nr; ++j)
      outs.push_back((partial ? ops[j].accT : storageT(ops[j].dt)) + "* __restrict__ out" + std::to_string(j));
    if (wavePerRow) {
      s << "  const int lane = threadIdx.x & 63;\n";
      s << "  const " << IT << " kk = (" << IT << ")blockIdx.x * 4 + (threadIdx.x >> 6);\n";
      s << "  if (kk >= " << Kn << ") return;\n";
      s << "  const " << IT << " r_begin = 0, r_end = " << vecs << ";\n  const int r_step = 64, r_tid = lane;\n";
    } else {
      // (measured: 11.2 us against 10.6 us for the sum of ten million floats with the contiguous chunks, so off unless asked for)
      static const bool interleave = getenv("MI355X_REDUCE_INTERLEAVE") && atoi(getenv("MI355X_REDUCE_INTERLEAVE")) != 0;
      s << "  const " << IT << " kk = (" << IT << ")blockIdx.x / " << P << ";\n";
      if (interleave && P > 1) {
        // the workgroups of a row walk it together, each taking every P-th block of 256 vectors: at any moment the grid
        // reads one contiguous stretch of memory, as a plain streaming kernel does
        s << "  const " << IT << " r_begin = ((" << IT << ")blockIdx.x % " << P << ") * 256;\n";
        s << "  const " << IT << " r_end = " << vecs << ";\n";
        s << "  const " << IT << " r_step = " << 256 * P << ";\n  const int r_tid = threadIdx.x;\n";
      } else {
        s << "  const " << IT << " chunk = (" << vecs << " + " << P << " - 1) / " << P << ";\n";
        s << "  const " << IT << " r_begin = ((" << IT << ")blockIdx.x % " << P << ") * chunk;\n";
        s << "  const " << IT << " r_end = r_begin + chunk < " << vecs << " ? r_begin + chunk : " << vecs << ";\n";
        s << "  const int r_step = 256, r_tid = threadIdx.x;\n";
      }
    }
    s << em.pre_;
    for (size_t j = 0; j < nr; ++j) s << "  " << ops[j].accT << " acc" << j << " = " << ops[j].identity << ";\n";
    s << "  #pragma unroll " << rowUnroll << "\n  for (" << IT << " rv = r_begin + r_tid; rv < r_end; rv += r_step) {\n";
    s << "    const " << IT << " rb = rv * " << V << ";\n";
    s << loopPre;
    s << "    #pragma unroll\n    for (int v = 0; v < " << V << "; ++v) {\n";
    s << em.body_.front();
    for (size_t j = 0; j < nr; ++j) s << "      acc" << j << " = " << ops[j].combine("acc" + std::to_string(j), vals[j]) << ";\n";
    s << "    }\n  }\n";
    // wavefront reduction
    for (size_t j = 0; j < nr; ++j) {
      s << "  #pragma unroll\n  for (int o = 32; o > 0; o >>= 1) acc" << j << " = "
        << ops[j].combine("acc" + std::to_string(j), shflXor(ops[j].accT, "acc" + std::to_string(j), "o")) << ";\n";
    }
    if (!wavePerRow) {
      for (size_t j = 0; j < nr; ++j) s << "  __shared__ " << (ops[j].accT == "bool" ? "int" : ops[j].accT) << " sm" << j << "[4];\n";
      s << "  if ((threadIdx.x & 63) == 0) {";
      for (size_t j = 0; j < nr; ++j) s << " sm" << j << "[threadIdx.x >> 6] = acc" << j << ";";
      s << " }\n  __syncthreads();\n  if (threadIdx.x != 0) return;\n";
      for (size_t j = 0; j < nr; ++j) {
        s << "  acc" << j << " = (" << ops[j].accT << ")sm" << j << "[0];\n";
        s << "  for (int w = 1; w < 4; ++w) acc" << j << " = " << ops[j].combine("acc" + std::to_string(j), "(" + ops[j].accT + ")sm" + std::to_string(j) + "[w]") << ";\n";
      }
    } else {
      s << "  if (lane != 0) return;\n";
    }
    for (size_t j = 0; j < nr; ++j) {
      if (partial) s << "  out" << j << "[kk * " << P << " + ((" << IT << ")blockIdx.x % " << P << ")] = acc" << j << ";\n";
      else {
        s << "  const " << ops[j].accT << " res" << j << " = " << roundTo(ops[j].dt, ops[j].combine(inits[j], "acc" + std::to_string(j))) << ";\n";
        s << "  out" << j << "[kk] = " << storeExpr(ops[j].dt, "res" + std::to_string(j)) << ";\n";
      }
    }
    // one pass: the lane that holds a finished result also computes the per-output values that need nothing else
    std::string header = kernelHeader(em.leaves_, outs);
    if (!partial && !epilogue.empty()) {
      for (size_t j = 0; j < nr; ++j) em.rowScalars_[reduces[j]->result()] = "res" + std::to_string(j);
      em.rowKept_ = kd;
      Index kidx = em.multiIndex(kd, keptShape);
      std::string savedPre2 = em.pre_;
      em.pre_.clear();
      em.forgetBodyValues();
      const size_t bodyMark = em.body_.front().size();
      std::vector<std::string> ev;
      for (auto* v : epilogue) ev.push_back(em.gen(v, kidx));
      s << em.pre_ << "  { const int v = 0; (void)v;\n" << em.body_.front().substr(bodyMark);
      em.pre_ = savedPre2;
      for (size_t q = 0; q < epilogue.size(); ++q) {
        s << "  outE" << q << "[kk] = " << storeExpr(epilogue[q]->type.dt, ev[q]) << ";\n";
        outs.push_back(storageT(epilogue[q]->type.dt) + "* __restrict__ outE" + std::to_string(q));
      }
      s << "  }\n";
      header = kernelHeader(em.leaves_, outs);
      fc.epilogueFused = true;
    }
    s << "}\n";
    Launch l;
    l.source = std::string(kPrelude) + header + " {\n" + s.str();
    l.grid[0] = (unsigned)(wavePerRow ? (Kn + 3) / 4 : Kn * P);
    l.block[0] = 256;
    for (auto* v : em.leaves_) { KArg a; a.kind = KArg::In; a.value = v; l.args.push_back(a); }
    std::vector<int64_t> workOff;
    int64_t wb = 0;
    for (size_t j = 0; j < nr; ++j) {
      KArg a;
      if (partial) {
        a.kind = KArg::Work;
        a.workOffset = wb;
        workOff.push_back(wb);
        wb += ((int64_t)P * Kn * 8 + 255) / 256 * 256;
      } else {
        a.kind = KArg::Out;
        a.value = reduces[j]->result();
      }
      l.args.push_back(a);
    }
    if (!partial) for (auto* v : epilogue) { KArg a; a.kind = KArg::Out; a.value = v; l.args.push_back(a); }
    fc.leaves = em.leaves_;
    fc.launches.push_back(std::move(l));
    if (partial) {
      std::vector<Value*> il;
      fc.launches.push_back(finalPass(P, Kn, workOff, il));
      fc.epilogueFused = !epilogue.empty();
      for (auto* v : il) if (std::find(fc.leaves.begin(), fc.leaves.end(), v) == fc.leaves.end()) fc.leaves.push_back(v);
      fc.workspaceBytes = wb;
    }
    return fc;
  }

  // ---- column style: lanes along the kept (contiguous) axis, rows split over
  // threadIdx.y and, when there are many rows, over blockIdx.y (partials).
  int V = 1;
  {
    int v = (int)std::min<size_t>(8, std::max<size_t>(1, 16 / std::max<size_t>(1, dtypeSize(x0->type.dt))));
    int64_t lastKept = keptShape.back();
    bool innerIsLastKept = keptDims.back() == inner;
    while (v > 1 && (!innerIsLastKept || lastKept % v != 0)) v >>= 1;
    V = v;
  }
  const bool onePass = Rn * Kn <= reduceOnePassLimit();
  if (onePass) while (V > 1 && Rn * Kn / V < kSpreadThreads) V >>= 1;   // small inputs: lanes before vectors, as in the loop kernels
  int64_t kvecs = (Kn + V - 1) / V;
  int TX = 1;
  while (TX < 64 && TX < kvecs) TX <<= 1;
  int TY = 256 / TX;
  int64_t gridX = (kvecs + TX - 1) / TX;
  int64_t P = 1;
  static const int colPerThread = getenv("MI355X_REDUCE_COL_PER_THREAD") ? atoi(getenv("MI355X_REDUCE_COL_PER_THREAD")) : 16;
  if (Rn > (int64_t)TY * 16) P = std::min<int64_t>((Rn + TY * colPerThread - 1) / (TY * colPerThread), std::max<int64_t>(1, 2048 / gridX));
  // a small input is cheaper to walk in one launch (a few dozen loads per lane) than to split over a second, dependent one
  if (Rn * Kn <= reduceOnePassLimit() && Rn <= (int64_t)TY * 128) P = 1;
  // one pass over few columns: narrower column tiles put more workgroups on the rows (64 x 1024: 32 workgroups of 32 row
  // lanes instead of 4 of 4), which matters when every element is a chain of its own
  if (P == 1) {
    const int64_t want = std::min<int64_t>(256, std::max<int64_t>(1, Rn * Kn / V / 512));   // about two visits per lane, a workgroup per compute unit at most
    while (TX > 8 && (kvecs + TX - 1) / TX < want && 256 / (TX / 2) <= Rn) TX >>= 1, TY = 256 / TX, gridX = (kvecs + TX - 1) / TX;
  }
  bool partial = P > 1;
  Emitter em(isLeaf, V, i64);
  IdxDim klin;
  klin.isConst = false; klin.base = "kb"; klin.coef = V > 1 ? 1 : 0; klin.mult = V;
  auto kd = em.delinearize(klin, keptShape);
  std::string savedPre = em.pre_;
  em.pre_.clear();
  IdxDim rlin;
  rlin.isConst = false; rlin.base = "rr"; rlin.coef = 0; rlin.mult = 1;
  auto rd = em.delinearize(rlin, redShape);
  std::vector<IdxDim> full(rank);
  for (size_t q = 0; q < keptDims.size(); ++q) full[keptDims[q]] = kd[q];
  for (size_t q = 0; q < redDims.size(); ++q) full[redDims[q]] = rd[q];
  Index idx = em.multiIndex(full, shape);
  std::vector<std::string> vals;
  for (auto* r : reduces) vals.push_back(em.gen(r->operands[0], idx));
  // values the caller wants in memory as well: every (row, column) is visited exactly once, so they are stored on the way
  for (size_t q = 0; q < sideStores.size(); ++q) {
    Value* sv = sideStores[q];
    if (sv->type.dims != shape) throw CompileError("codegen: side store of another shape");
    const std::string e = em.gen(sv, idx);
    em.body("side" + std::to_string(q) + "[" + em.dimExpr(em.linearize(full, shape)) + "] = " + storeExpr(sv->type.dt, e) + ";");
  }
  std::string loopPre = em.pre_;
  em.pre_ = savedPre;
  std::vector<std::string> inits;
  for (auto* r : reduces) inits.push_back(em.gen(r->operands[1], em.multiIndex({}, {})));

  std::ostringstream s;   // body; the header follows once an epilogue has named its inputs
  std::vector<std::string> outs;
  for (size_t j = 0; j < nr; ++j)
    outs.push_back((partial ? ops[j].accT : storageT(ops[j].dt)) + "* __restrict__ out" + std::to_string(j));
  for (size_t q = 0; q < sideStores.size(); ++q) outs.push_back(storageT(sideStores[q]->type.dt) + "* __restrict__ side" + std::to_string(q));
  s << "  const int tx = threadIdx.x % " << TX << ", ty = threadIdx.x / " << TX << ";\n";
  s << "  const " << IT << " kb = ((" << IT << ")blockIdx.x * " << TX << " + tx) * " << V << ";\n";
  s << "  const bool active = kb < " << Kn << ";\n";
  s << "  const " << IT << " chunk = (" << Rn << " + " << P << " - 1) / " << P << ";\n";
  // (a single-pass kernel names no second grid index, so that it can share a launch with its neighbours)
  s << "  const " << IT << " r_begin = " << (partial ? "(" + IT + ")blockIdx.y * chunk" : std::string("0")) << ";\n";
  s << "  const " << IT << " r_end = r_begin + chunk < " << Rn << " ? r_begin + chunk : " << Rn << ";\n";
  for (size_t j = 0; j < nr; ++j) {
    s << "  " << ops[j].accT << " acc" << j << "[" << V << "];\n";
    s << "  #pragma unroll\n  for (int v = 0; v < " << V << "; ++v) acc" << j << "[v] = " << ops[j].identity << ";\n";
  }
  s << "  if (active) {\n";
  s << em.pre_;
  s << "  #pragma unroll 4\n  for (" << IT << " rr = r_begin + ty; rr < r_end; rr += " << TY << ") {\n";
  s << loopPre;
  s << "    #pragma unroll\n    for (int v = 0; v < " << V << "; ++v) {\n";
  s << em.body_.front();
  for (size_t j = 0; j < nr; ++j) s << "      acc" << j << "[v] = " << ops[j].combine("acc" + std::to_string(j) + "[v]", vals[j]) << ";\n";
  s << "    }\n  }\n  }\n";
  if (TY > 1) {
    for (size_t j = 0; j < nr; ++j) {
      std::string ST = ops[j].accT == "bool" ? "int" : ops[j].accT;
      s << "  __shared__ " << ST << " sm" << j << "[" << TY << "][" << TX * V << " + 1];\n";
      s << "  #pragma unroll\n  for (int v = 0; v < " << V << "; ++v) sm" << j << "[ty][tx * " << V << " + v] = acc" << j << "[v];\n";
    }
    s << "  __syncthreads();\n  if (ty != 0 || !active) return;\n";
    for (size_t j = 0; j < nr; ++j) {
      s << "  for (int y = 1; y < " << TY << "; ++y) {\n    #pragma unroll\n    for (int v = 0; v < " << V << "; ++v) acc" << j << "[v] = "
        << ops[j].combine("acc" + std::to_string(j) + "[v]", "(" + ops[j].accT + ")sm" + std::to_string(j) + "[y][tx * " + std::to_string(V) + " + v]") << ";\n  }\n";
    }
  } else {
    s << "  if (!active) return;\n";
  }
  const bool epilogueHere = !partial && !epilogue.empty();
  if (epilogueHere) {
    // a single pass holds the finished results: per-output values that only need those are computed by the lane that holds them
    s << "  #pragma unroll\n  for (int v = 0; v < " << V << "; ++v) {\n    const " << IT << " kk = kb + v;\n";
    for (size_t j = 0; j < nr; ++j) {
      s << "    const " << ops[j].accT << " res" << j << " = " << roundTo(ops[j].dt, ops[j].combine(inits[j], "acc" + std::to_string(j) + "[v]")) << ";\n";
      s << "    out" << j << "[kk] = " << storeExpr(ops[j].dt, "res" + std::to_string(j)) << ";\n";
      em.rowScalars_[reduces[j]->result()] = "res" + std::to_string(j);
    }
    IdxDim klin2;
    klin2.isConst = false; klin2.base = "kk"; klin2.coef = 0; klin2.mult = 1;
    const std::string keepPre = em.pre_;
    em.pre_.clear();
    em.forgetBodyValues();
    const size_t bodyMark = em.body_.front().size();
    auto kd2 = em.delinearize(klin2, keptShape);
    em.rowKept_ = kd2;
    Index kidx = em.multiIndex(kd2, keptShape);
    std::vector<std::string> ev;
    for (auto* v : epilogue) ev.push_back(em.gen(v, kidx));
    s << em.pre_ << em.body_.front().substr(bodyMark);
    em.pre_ = keepPre;
    for (size_t q = 0; q < epilogue.size(); ++q) {
      s << "    outE" << q << "[kk] = " << storeExpr(epilogue[q]->type.dt, ev[q]) << ";\n";
      outs.push_back(storageT(epilogue[q]->type.dt) + "* __restrict__ outE" + std::to_string(q));
    }
    s << "  }\n";
    fc.epilogueFused = true;
  } else {
    for (size_t j = 0; j < nr; ++j) {
      s << "  #pragma unroll\n  for (int v = 0; v < " << V << "; ++v) ";
      if (partial) s << "out" << j << "[(kb + v) * " << P << " + (" << IT << ")blockIdx.y] = acc" << j << "[v];\n";
      else s << "out" << j << "[kb + v] = " << storeExpr(ops[j].dt, roundTo(ops[j].dt, ops[j].combine(inits[j], "acc" + std::to_string(j) + "[v]"))) << ";\n";
    }
  }
  s << "}\n";
  Launch l;
  l.source = std::string(kPrelude) + kernelHeader(em.leaves_, outs) + " {\n" + s.str();
  l.grid[0] = (unsigned)gridX;
  l.grid[1] = (unsigned)P;
  l.block[0] = 256;
  for (auto* v : em.leaves_) { KArg a; a.kind = KArg::In; a.value = v; l.args.push_back(a); }
  std::vector<int64_t> workOff;
  int64_t wb = 0;
  for (size_t j = 0; j < nr; ++j) {
    KArg a;
    if (partial) {
      a.kind = KArg::Work;
      a.workOffset = wb;
      workOff.push_back(wb);
      wb += ((int64_t)P * Kn * 8 + 255) / 256 * 256;
    } else {
      a.kind = KArg::Out;
      a.value = reduces[j]->result();
    }
    l.args.push_back(a);
  }
  for (auto* sv : sideStores) { KArg a; a.kind = KArg::Out; a.value = sv; l.args.push_back(a); }
  if (epilogueHere) for (auto* v : epilogue) { KArg a; a.kind = KArg::Out; a.value = v; l.args.push_back(a); }
  fc.sideStored = !sideStores.empty();
  fc.leaves = em.leaves_;
  fc.launches.push_back(std::move(l));
  if (partial) {
    std::vector<Value*> il;
    fc.launches.push_back(finalPass(P, Kn, workOff, il));
      fc.epilogueFused = !epilogue.empty();
    for (auto* v : il) if (std::find(fc.leaves.begin(), fc.leaves.end(), v) == fc.leaves.end()) fc.leaves.push_back(v);
    fc.workspaceBytes = wb;
  }
  return fc;
}

// ------------------------------------------------------------ reductions with any body
// stablehlo.reduce over n inputs with an arbitrary reducer region (argmax / argmin as JAX
// lowers them: a (value, index) pair with a compare-select body; reference: the argmax/argmin
// pattern of ops/reduction.cc:83-162).  The region is generated as straight-line code over
// the accumulator tuple.  One wavefront per output: lanes stride over the reduced elements,
// then a butterfly over the tuple.  Every lane starts from the init tuple, which the
// operation allows to be combined any number of times.
FusedCode generateRegionReduce(Op* reduce, const LeafPredicate& isLeaf) {
  const size_t n = reduce->operands.size() / 2;
  if (n == 0 || reduce->operands.size() != 2 * n || reduce->results.size() != n || reduce->regions.size() != 1)
    throw CompileError("stablehlo.reduce: malformed operands");
  Region& body = *reduce->regions[0];
  if (body.args.size() != 2 * n || !body.terminator() || body.terminator()->operands.size() != n)
    throw CompileError("stablehlo.reduce: the reducer region does not match the operands");
  for (auto& op : body.ops)
    if (op->name != "return" && (!isFusibleOp(*op) || op->results.size() != 1 || !op->regions.empty()))
      throw CompileError("stablehlo.reduce: reducer body op stablehlo." + op->name + " is not supported");
  Value* x0 = reduce->operands[0];
  const std::vector<int64_t>& shape = x0->type.dims;
  for (size_t j = 1; j < n; ++j)
    if (reduce->operands[j]->type.dims != shape) throw CompileError("stablehlo.reduce: inputs of different shapes");
  int rank = (int)shape.size();
  std::vector<int64_t> rdims = reduce->ints("dimensions");
  std::sort(rdims.begin(), rdims.end());
  std::vector<bool> isRed(rank, false);
  for (auto d : rdims) isRed[d] = true;
  std::vector<int64_t> keptShape, redShape;
  std::vector<int> keptDims, redDims;
  for (int d = 0; d < rank; ++d) {
    if (isRed[d]) { redShape.push_back(shape[d]); redDims.push_back(d); }
    else { keptShape.push_back(shape[d]); keptDims.push_back(d); }
  }
  int64_t Kn = 1, Rn = 1;
  for (auto d : keptShape) Kn *= d;
  for (auto d : redShape) Rn *= d;
  const bool i64 = x0->type.numel() >= (int64_t(1) << 31) - 16;
  const std::string IT = i64 ? "i64" : "int";

  Emitter em(isLeaf, 1, i64);
  IdxDim klin;
  klin.isConst = false; klin.base = "kk"; klin.coef = 0; klin.mult = 1;
  auto kd = em.delinearize(klin, keptShape);
  std::string savedPre = em.pre_;
  em.pre_.clear();
  IdxDim rlin;
  rlin.isConst = false; rlin.base = "rb"; rlin.coef = 0; rlin.mult = 1;
  auto rd = em.delinearize(rlin, redShape);
  std::vector<IdxDim> full(rank);
  for (size_t q = 0; q < keptDims.size(); ++q) full[keptDims[q]] = kd[q];
  for (size_t q = 0; q < redDims.size(); ++q) full[redDims[q]] = rd[q];
  Index idx = em.multiIndex(full, shape);
  std::vector<std::string> vals;
  for (size_t j = 0; j < n; ++j) vals.push_back(em.gen(reduce->operands[j], idx));
  std::string loopPre = em.pre_;
  em.pre_ = savedPre;
  std::vector<std::string> inits;
  for (size_t j = 0; j < n; ++j) inits.push_back(em.gen(reduce->operands[n + j], em.multiIndex({}, {})));

  std::vector<DType> dts;
  std::vector<std::string> accT;
  for (size_t j = 0; j < n; ++j) { dts.push_back(reduce->results[j]->type.dt); accT.push_back(computeT(dts[j])); }

  // (acc tuple) = body(acc tuple, other tuple), as a block of straight-line code
  int site = 0;
  auto combine = [&](const std::vector<std::string>& other, const std::string& indent) {
    Emitter b(isLeaf, 1, i64);
    b.shareLeavesFrom(em);
    b.startTemporariesAt(100000 * (site + 1));
    for (size_t j = 0; j < n; ++j) {
      b.rowScalars_[body.args[j].get()] = "acc" + std::to_string(j);
      b.rowScalars_[body.args[n + j].get()] = other[j];
    }
    std::vector<std::string> res;
    for (size_t j = 0; j < n; ++j) res.push_back(b.gen(body.terminator()->operands[j], b.multiIndex({}, {})));
    if (b.leaves_.size() != em.leaves_.size()) throw CompileError("stablehlo.reduce: the reducer region reads values defined outside it");
    std::ostringstream o;
    o << indent << "{\n" << b.pre_;
    for (size_t j = 0; j < n; ++j) o << indent << "  const " << accT[j] << " nx" << site << "_" << j << " = " << roundTo(dts[j], res[j]) << ";\n";
    for (size_t j = 0; j < n; ++j) o << indent << "  acc" << j << " = nx" << site << "_" << j << ";\n";
    o << indent << "}\n";
    ++site;
    return o.str();
  };

  std::ostringstream s;
  s << "  const int lane = threadIdx.x & 63;\n";
  s << "  const " << IT << " kk = (" << IT << ")blockIdx.x * 4 + (threadIdx.x >> 6);\n";
  s << "  if (kk >= " << Kn << ") return;\n";
  s << em.pre_;
  for (size_t j = 0; j < n; ++j) s << "  " << accT[j] << " acc" << j << " = " << inits[j] << ";\n";
  s << "  for (" << IT << " rb = lane; rb < " << Rn << "; rb += 64) {\n";
  s << loopPre;
  s << "    { const int v = 0; (void)v;\n" << em.body_.front();
  s << combine(vals, "    ");
  s << "    }\n  }\n";
  s << "  #pragma unroll\n  for (int o = 32; o > 0; o >>= 1) {\n";
  std::vector<std::string> peers;
  for (size_t j = 0; j < n; ++j) {
    s << "    const " << accT[j] << " pr" << j << " = " << shflXor(accT[j], "acc" + std::to_string(j), "o") << ";\n";
    peers.push_back("pr" + std::to_string(j));
  }
  s << combine(peers, "    ");
  s << "  }\n";
  s << "  if (lane != 0) return;\n";
  for (size_t j = 0; j < n; ++j) s << "  out" << j << "[kk] = " << storeExpr(dts[j], "acc" + std::to_string(j)) << ";\n";
  s << "}\n";

  std::vector<std::string> outs;
  for (size_t j = 0; j < n; ++j) outs.push_back(storageT(dts[j]) + "* __restrict__ out" + std::to_string(j));
  FusedCode fc;
  Launch l;
  l.source = std::string(kPrelude) + kernelHeader(em.leaves_, outs) + " {\n" + s.str();
  l.grid[0] = (unsigned)((Kn + 3) / 4);
  l.block[0] = 256;
  for (auto* v : em.leaves_) { KArg a; a.kind = KArg::In; a.value = v; l.args.push_back(a); }
  for (size_t j = 0; j < n; ++j) { KArg a; a.kind = KArg::Out; a.value = reduce->results[j].get(); l.args.push_back(a); }
  fc.leaves = em.leaves_;
  fc.launches.push_back(std::move(l));
  return fc;
}

// ------------------------------------------------------------------ row programs
// One kernel per group of rows: every phase walks the row once (from HBM the first time, from
// cache afterwards), phase p may use the reductions finished in phases < p, and the last walk
// stores the elementwise results.  Softmax is (max | sum of exp | divide), LayerNorm is
// (sum, sum of squares | normalise); HBM traffic is one read and one write of the tensor.
FusedCode generateRowProgram(const RowProgram& rp, const LeafPredicate& isLeaf) {
  Op* r0 = rp.phases.at(0).at(0);
  Value* x0 = r0->operands[0];
  const std::vector<int64_t>& shape = x0->type.dims;
  int rank = (int)shape.size();
  std::vector<int64_t> rdims = r0->ints("dimensions");
  std::sort(rdims.begin(), rdims.end());
  std::vector<bool> isRed(rank, false);
  for (auto d : rdims) isRed[d] = true;
  std::vector<int64_t> keptShape, redShape;
  std::vector<int> keptDims, redDims;
  for (int d = 0; d < rank; ++d) {
    if (isRed[d]) { redShape.push_back(shape[d]); redDims.push_back(d); }
    else { keptShape.push_back(shape[d]); keptDims.push_back(d); }
  }
  for (size_t q = 0; q < redDims.size(); ++q)
    if (redDims[q] != rank - (int)redDims.size() + (int)q) throw CompileError("row program: reduced dims are not the trailing dims");
  int64_t Kn = 1, Rn = 1;
  for (auto d : keptShape) Kn *= d;
  for (auto d : redShape) Rn *= d;

  std::unordered_set<Value*> inGroup;
  std::vector<Op*> reduces;
  for (auto& ph : rp.phases) for (auto* r : ph) { reduces.push_back(r); inGroup.insert(r->result()); }
  for (auto* v : rp.fullRoots) inGroup.insert(v);
  for (auto* v : rp.keptRoots) inGroup.insert(v);
  LeafPredicate inner = [&](Value* v) { return !inGroup.count(v) && isLeaf(v); };

  int V = 8;
  for (auto* r : reduces) V = std::min(V, pickVector(r->operands[0]->type));
  for (auto* v : rp.fullRoots) V = std::min(V, pickVector(v->type));
  while (V > 1 && (redShape.empty() || redShape.back() % V != 0)) V >>= 1;
  if (Rn < 64 * V) V = 1;
  const int64_t vecs = (Rn + V - 1) / V;
  const bool wavePerRow = vecs <= 256;
  const bool i64 = (double)Kn * (double)Rn >= 2147483000.0;
  const std::string IT = i64 ? "i64" : "int";

  // short rows are walked by fully unrolled loops: the compiler then keeps the row (and pure
  // functions of it) in registers from one phase to the next instead of re-reading it
  const int64_t walks = (vecs + (wavePerRow ? 64 : 256) - 1) / (wavePerRow ? 64 : 256);
  const int walkUnroll = walks <= 8 ? (int)walks : 4;
  // Rows of at most eight walks: the walks are unrolled with the walk number a constant, and what one walk
  // computed per element (loaded operands, exponentials, differences) is kept in registers for the later
  // walks that need it instead of being loaded or computed again.
  static const bool carryOff = getenv("MI355X_ROW_CARRY") && atoi(getenv("MI355X_ROW_CARRY")) == 0;
  const bool carry = !carryOff && walks <= 8 && walks * V <= 32;
  const int maxCarried = 4;
  struct Kept { std::string name, expr, type; size_t phase; bool used; };
  std::unordered_map<std::string, Kept> kept;   // by "value|index" key
  int keptNames = 0, keptUsed = 0;
  std::unordered_map<Value*, std::string> scalars;
  std::unordered_map<std::string, std::string> rcps;
  std::ostringstream b;   // kernel body; the header needs the final leaf list
  if (wavePerRow) {
    b << "  const int r_tid = threadIdx.x & 63, r_step = 64;\n";
    b << "  const " << IT << " kk = (" << IT << ")blockIdx.x * 4 + (threadIdx.x >> 6);\n";
    b << "  if (kk >= " << Kn << ") return;\n";
  } else {
    b << "  const int r_tid = threadIdx.x, r_step = 256;\n";
    b << "  const " << IT << " kk = (" << IT << ")blockIdx.x;\n";
  }
  b << "  const int r_end = " << vecs << ";\n";
  std::vector<RedOp> ops;
  for (size_t i = 0; i < reduces.size(); ++i) {
    ops.push_back(makeRedOp(*reduces[i]));
    b << "  " << ops[i].accT << " red" << i << ";\n";
    if (ops[i].accT == "float") b << "  float rcp" << i << ";\n";
  }
  auto walkOpen = [&](std::ostringstream& o) {
    if (carry) {
      o << "  #pragma unroll\n  for (int it = 0; it < " << walks << "; ++it) {\n";
      o << "    const int rv = r_tid + it * r_step;\n";
      o << "    if (it + 1 < " << walks << " || rv < r_end) {\n";
    } else {
      o << "  #pragma unroll " << walkUnroll << "\n  for (int rv = r_tid; rv < r_end; rv += r_step) {\n";
    }
  };
  auto walkClose = [&](std::ostringstream& o) { o << (carry ? "    }\n  }\n" : "  }\n"); };

  // per phase: a fresh emitter (own temporaries inside its own scope) over the shared leaf list
  std::unique_ptr<Emitter> prev;
  auto newEmitter = [&]() {
    auto em = std::make_unique<Emitter>(inner, V, i64);
    if (prev) em->shareLeavesFrom(*prev);
    em->rowScalars_ = scalars;
    em->rowRcp_ = rcps;
    if (carry) {
      for (auto& kv : kept) {
        em->seeded_[kv.first] = kv.second.name + "[it][v]";
        em->bodyNames_.insert(kv.second.name);
      }
      em->seededCap_ = maxCarried - keptUsed;
    }
    return em;
  };
  // index of element (row kk, position rb + v) and of the row itself
  auto rowIndex = [&](Emitter& em, std::string& loopPre, Index& full, Index& keptIdx) {
    IdxDim klin;
    klin.isConst = false; klin.base = "kk"; klin.coef = 0; klin.mult = 1;
    auto kd = em.delinearize(klin, keptShape);
    em.rowKept_ = kd;
    keptIdx = em.multiIndex(kd, keptShape);
    std::string savedPre = em.pre_;
    em.pre_.clear();
    IdxDim rlin;
    rlin.isConst = false; rlin.base = "rb"; rlin.coef = V > 1 ? 1 : 0; rlin.mult = V;
    auto rd = em.delinearize(rlin, redShape);
    std::vector<IdxDim> dims(rank);
    for (size_t q = 0; q < keptDims.size(); ++q) dims[keptDims[q]] = kd[q];
    for (size_t q = 0; q < redDims.size(); ++q) dims[redDims[q]] = rd[q];
    full = em.multiIndex(dims, shape);
    loopPre = em.pre_;
    em.pre_ = savedPre;
  };
  // the text of a walk is final only when the later walks have said what they want kept
  std::vector<std::string> walkHead, walkTail, keepStores;
  // after a walk was generated: note what later walks took from registers, offer what this one computed
  auto settle = [&](Emitter& em, const Index& full, size_t phase) {
    if (!carry) return;
    std::vector<std::string> usedKeys(em.seededUsed_.begin(), em.seededUsed_.end());
    std::sort(usedKeys.begin(), usedKeys.end());
    for (auto& key : usedKeys) {
      Kept& k = kept.at(key);
      if (k.used) continue;
      k.used = true;
      ++keptUsed;
      keepStores[k.phase] += "      " + k.name + "[it][v] = " + k.expr + ";\n";
    }
    const std::string suffix = "|" + full.sig;
    std::vector<std::pair<std::string, std::string>> fresh(em.unguardedValues().begin(), em.unguardedValues().end());
    std::sort(fresh.begin(), fresh.end());   // names must not depend on hash order: the source text is the cache key
    for (auto& kv : fresh) {
      const std::string& key = kv.first;
      if (key.size() <= suffix.size() || key.compare(key.size() - suffix.size(), suffix.size(), suffix) != 0 || kept.count(key)) continue;
      auto vi = em.keyValue_.find(key);
      if (vi == em.keyValue_.end()) continue;
      Value* v = vi->second;
      if (v->type.dims != shape || scalars.count(v)) continue;
      if (v->def && (v->def->name == "constant" || v->def->name == "iota" || v->def->name == "broadcast_in_dim")) continue;
      kept[key] = Kept{"cr" + std::to_string(keptNames++), kv.second, computeT(v->type.dt), phase, false};
    }
  };

  size_t base = 0;
  for (size_t p = 0; p < rp.phases.size(); ++p) {
    auto& ph = rp.phases[p];
    auto em = newEmitter();
    std::string idxPre;
    Index full, keptIdx;
    rowIndex(*em, idxPre, full, keptIdx);
    std::string savedPre = em->pre_;
    em->pre_.clear();
    std::vector<std::string> vals;
    for (auto* r : ph) vals.push_back(em->gen(r->operands[0], full));
    std::string loopPre = idxPre + em->pre_;
    em->pre_ = savedPre;
    std::vector<std::string> inits;
    for (auto* r : ph) inits.push_back(em->gen(r->operands[1], em->multiIndex({}, {})));
    std::ostringstream h, t;
    h << "  {\n" << em->pre_;
    for (size_t j = 0; j < ph.size(); ++j) h << "  " << ops[base + j].accT << " acc" << j << " = " << ops[base + j].identity << ";\n";
    walkOpen(h);
    h << "    const int rb = rv * " << V << ";\n" << loopPre;
    h << "    #pragma unroll\n    for (int v = 0; v < " << V << "; ++v) {\n" << em->body_.front();
    for (size_t j = 0; j < ph.size(); ++j) t << "      acc" << j << " = " << ops[base + j].combine("acc" + std::to_string(j), vals[j]) << ";\n";
    t << "    }\n";
    walkClose(t);
    for (size_t j = 0; j < ph.size(); ++j) {
      const RedOp& o = ops[base + j];
      std::string a = "acc" + std::to_string(j);
      t << "  #pragma unroll\n  for (int o = 32; o > 0; o >>= 1) " << a << " = " << o.combine(a, shflXor(o.accT, a, "o")) << ";\n";
      if (!wavePerRow) {
        std::string ST = o.accT == "bool" ? "int" : o.accT;
        std::string sm = "sm" + std::to_string(base + j);
        t << "  __shared__ " << ST << " " << sm << "[4];\n";
        t << "  if ((threadIdx.x & 63) == 0) " << sm << "[threadIdx.x >> 6] = " << a << ";\n  __syncthreads();\n";
        t << "  " << a << " = (" << o.accT << ")" << sm << "[0];\n";
        t << "  for (int w = 1; w < 4; ++w) " << a << " = " << o.combine(a, "(" + o.accT + ")" + sm + "[w]") << ";\n";
      }
      t << "  red" << (base + j) << " = " << roundTo(o.dt, o.combine(inits[j], a)) << ";\n";
      if (o.accT == "float") t << "  rcp" << (base + j) << " = 1.f / red" << (base + j) << ";\n";
    }
    t << "  }\n";
    walkHead.push_back(h.str());
    walkTail.push_back(t.str());
    keepStores.emplace_back();
    settle(*em, full, p);
    for (size_t j = 0; j < ph.size(); ++j) {
      scalars[ph[j]->result()] = "red" + std::to_string(base + j);
      if (ops[base + j].accT == "float") rcps["red" + std::to_string(base + j)] = "rcp" + std::to_string(base + j);
    }
    base += ph.size();
    prev = std::move(em);
  }

  // last walk: elementwise results of the full shape, then the per-row results
  {
    auto em = newEmitter();
    std::string idxPre;
    Index full, keptIdx;
    rowIndex(*em, idxPre, full, keptIdx);
    // the per-row results first, ahead of the walk: a full-shape result that reads one of them (through a broadcast)
    // then finds it declared where the store after the walk can see it too
    std::vector<std::string> kvals;
    for (auto* v : rp.keptRoots) kvals.push_back(em->gen(v, keptIdx));
    std::string savedPre = em->pre_;
    em->pre_.clear();
    std::vector<std::string> vals;
    for (auto* v : rp.fullRoots) vals.push_back(em->gen(v, full));
    std::string loopPre = idxPre + em->pre_;
    em->pre_ = savedPre;
    std::ostringstream h, t;
    h << "  {\n" << em->pre_;
    if (!rp.fullRoots.empty()) {
      walkOpen(h);
      h << "    const int rb = rv * " << V << ";\n" << loopPre;
      for (size_t j = 0; j < rp.fullRoots.size(); ++j) h << "    Vec<" << storageT(rp.fullRoots[j]->type.dt) << ", " << V << "> ov" << j << ";\n";
      h << "    #pragma unroll\n    for (int v = 0; v < " << V << "; ++v) {\n" << em->body_.front();
      for (size_t j = 0; j < rp.fullRoots.size(); ++j) h << "      ov" << j << ".e[v] = " << storeExpr(rp.fullRoots[j]->type.dt, vals[j]) << ";\n";
      h << "    }\n";
      for (size_t j = 0; j < rp.fullRoots.size(); ++j)
        h << "    *(Vec<" << storageT(rp.fullRoots[j]->type.dt) << ", " << V << ">*)(outF" << j << " + (" << IT << ")kk * " << Rn << " + rb) = ov" << j << ";\n";
      walkClose(h);
    }
    h << "  if (r_tid == 0) {\n";
    for (size_t j = 0; j < rp.keptRoots.size(); ++j) h << "    outK" << j << "[kk] = " << storeExpr(rp.keptRoots[j]->type.dt, kvals[j]) << ";\n";
    for (size_t i = 0; i < reduces.size(); ++i) h << "    outR" << i << "[kk] = " << storeExpr(ops[i].dt, "red" + std::to_string(i)) << ";\n";
    h << "  }\n  }\n";
    walkHead.push_back(h.str());
    walkTail.push_back("");
    keepStores.emplace_back();
    settle(*em, full, rp.phases.size());
    prev = std::move(em);
  }
  for (auto& kv : kept)
    if (kv.second.used) b << "  " << kv.second.type << " " << kv.second.name << "[" << walks << "][" << V << "];\n";
  for (size_t p = 0; p < walkHead.size(); ++p) b << walkHead[p] << keepStores[p] << walkTail[p];

  std::vector<std::string> outs;
  for (size_t j = 0; j < rp.fullRoots.size(); ++j) outs.push_back(storageT(rp.fullRoots[j]->type.dt) + "* __restrict__ outF" + std::to_string(j));
  for (size_t j = 0; j < rp.keptRoots.size(); ++j) outs.push_back(storageT(rp.keptRoots[j]->type.dt) + "* __restrict__ outK" + std::to_string(j));
  for (size_t i = 0; i < reduces.size(); ++i) outs.push_back(storageT(ops[i].dt) + "* __restrict__ outR" + std::to_string(i));
  if (prev->leaves_.size() + outs.size() > 60) throw CompileError("row program: too many kernel arguments");
  std::ostringstream s;
  s << kPrelude << kernelHeader(prev->leaves_, outs) << " {\n" << b.str() << "}\n";
  FusedCode fc;
  Launch l;
  l.source = s.str();
  l.grid[0] = (unsigned)(wavePerRow ? (Kn + 3) / 4 : Kn);
  l.block[0] = 256;
  for (auto* v : prev->leaves_) { KArg a; a.kind = KArg::In; a.value = v; l.args.push_back(a); }
  for (auto* v : rp.fullRoots) { KArg a; a.kind = KArg::Out; a.value = v; l.args.push_back(a); }
  for (auto* v : rp.keptRoots) { KArg a; a.kind = KArg::Out; a.value = v; l.args.push_back(a); }
  for (auto* r : reduces) { KArg a; a.kind = KArg::Out; a.value = r->result(); l.args.push_back(a); }
  fc.leaves = prev->leaves_;
  fc.launches.push_back(std::move(l));
  return fc;
}
// stablehlo.sort: one workgroup per slice along the sorted dim.  The operands of the slice are staged in LDS
// and a permutation is sorted by a bitonic network whose order is "comparator(a, b), else not comparator(b, a)
// and a came first", a strict total order, so the result is the stable sort whatever network produces it
// (reference: src/pjrt_plugin/ops/sort_fft_complex.cc:145-216, which sorts by the first operand only; here the
// comparator region itself is compiled, so multi-key and custom orders work).
int64_t sortLdsBytes(Op* sort) {
  int64_t L = sort->operands[0]->type.dims.empty() ? 1 : sort->operands[0]->type.dims[(size_t)sort->integer("dimension")];
  int64_t P = 1;
  while (P < L) P <<= 1;
  int64_t per = 4;
  for (auto* o : sort->operands) per += (int64_t)dtypeSize(o->type.dt);
  return P * per;
}

FusedCode generateSortKernel(Op* sort, const LeafPredicate& isLeaf) {
  const size_t n = sort->operands.size();
  if (n == 0 || sort->results.size() != n || sort->regions.size() != 1) throw CompileError("stablehlo.sort: malformed operands");
  Region& body = *sort->regions[0];
  if (body.args.size() != 2 * n || !body.terminator() || body.terminator()->operands.size() != 1)
    throw CompileError("stablehlo.sort: the comparator region does not match the operands");
  for (auto& op : body.ops)
    if (op->name != "return" && (!isFusibleOp(*op) || op->results.size() != 1 || !op->regions.empty()))
      throw CompileError("stablehlo.sort: comparator op stablehlo." + op->name + " is not supported");
  const TensorType& t0 = sort->operands[0]->type;
  for (auto* o : sort->operands) if (o->type.dims != t0.dims) throw CompileError("stablehlo.sort: operands of different shapes");
  const int rank = t0.rank();
  int64_t dim = rank == 0 ? 0 : sort->integer("dimension");
  if (dim < 0) dim += rank;
  int64_t L = rank == 0 ? 1 : t0.dims[(size_t)dim], inner = 1, outer = 1;
  for (int d = 0; d < rank; ++d) { if (d < dim) outer *= t0.dims[(size_t)d]; if (d > dim) inner *= t0.dims[(size_t)d]; }
  int64_t P = 1;
  while (P < L) P <<= 1;
  // slices too long for LDS are sorted in place in a workspace by the same network, one workgroup per slice
  // (values are read from the operands through the permutation; slower, but any length works)
  const bool inLds = sortLdsBytes(sort) <= 60 * 1024;
  if (t0.numel() >= (int64_t(1) << 31) || outer * inner * P >= (int64_t(1) << 31)) throw CompileError("stablehlo.sort: tensor too large");

  // comparator as straight-line code over named scalars
  Emitter b(isLeaf, 1, false);
  for (size_t j = 0; j < n; ++j) {
    b.rowScalars_[body.args[2 * j].get()] = "ca" + std::to_string(j);
    b.rowScalars_[body.args[2 * j + 1].get()] = "cb" + std::to_string(j);
  }
  std::string res = b.gen(body.terminator()->operands[0], b.multiIndex({}, {}));
  if (!b.leaves_.empty()) throw CompileError("stablehlo.sort: the comparator reads values defined outside it");

  std::ostringstream s;
  s << "  const int row = blockIdx.x;\n";
  s << "  const int base = (row / " << inner << ") * " << (L * inner) << " + (row % " << inner << ");\n";
  if (inLds) {
    for (size_t j = 0; j < n; ++j) s << "  __shared__ " << storageT(sort->operands[j]->type.dt) << " sv" << j << "[" << P << "];\n";
    s << "  __shared__ int perm[" << P << "];\n";
  } else {
    s << "  int* perm = work + (long long)row * " << P << ";\n";
  }
  s << "  for (int e = threadIdx.x; e < " << P << "; e += 256) {\n";
  s << "    perm[e] = e;\n";
  if (inLds) {
    s << "    if (e < " << L << ") {\n";
    for (size_t j = 0; j < n; ++j) s << "      sv" << j << "[e] = in" << j << "[base + e * " << inner << "];\n";
    s << "    }\n";
  }
  s << "  }\n  __syncthreads();\n";
  auto elem = [&](size_t j, const std::string& i) {
    return inLds ? "sv" + std::to_string(j) + "[" + i + "]" : "in" + std::to_string(j) + "[base + " + i + " * " + std::to_string(inner) + "]";
  };
  // before(a, b): a sorts strictly before b
  s << "  auto cmp = [&](int a, int b) -> bool {\n";
  for (size_t j = 0; j < n; ++j) {
    DType dt = sort->operands[j]->type.dt;
    s << "    const " << computeT(dt) << " ca" << j << " = " << loadExpr(dt, elem(j, "a")) << ";\n";
    s << "    const " << computeT(dt) << " cb" << j << " = " << loadExpr(dt, elem(j, "b")) << ";\n";
  }
  s << "    const int v = 0; (void)v;\n";
  s << b.pre_;
  s << "    return " << res << ";\n  };\n";
  s << "  auto before = [&](int a, int b) -> bool {\n";
  s << "    if (a >= " << L << " || b >= " << L << ") return a < b;   // padding sorts last\n";
  s << "    if (cmp(a, b)) return true;\n";
  s << "    if (cmp(b, a)) return false;\n";
  s << "    return a < b;\n  };\n";
  s << "  for (int k = 2; k <= " << P << "; k <<= 1) {\n";
  s << "    for (int j = k >> 1; j > 0; j >>= 1) {\n";
  s << "      for (int t = threadIdx.x; t < " << (P / 2) << "; t += 256) {\n";
  s << "        const int i = ((t / j) * 2 * j) + (t % j), l = i + j;\n";
  s << "        const int a = perm[i], c = perm[l];\n";
  s << "        const bool up = (i & k) == 0;\n";
  s << "        if (up ? before(c, a) : before(a, c)) { perm[i] = c; perm[l] = a; }\n";
  s << "      }\n      __syncthreads();\n    }\n  }\n";
  s << "  for (int e = threadIdx.x; e < " << L << "; e += 256) {\n";
  s << "    const int src = perm[e];\n";
  for (size_t j = 0; j < n; ++j) s << "    out" << j << "[base + e * " << inner << "] = " << elem(j, "src") << ";\n";
  s << "  }\n}\n";

  std::vector<Value*> leaves(sort->operands.begin(), sort->operands.end());
  std::vector<std::string> outs;
  for (size_t j = 0; j < n; ++j) outs.push_back(storageT(sort->results[j]->type.dt) + "* __restrict__ out" + std::to_string(j));
  if (!inLds) outs.push_back("int* __restrict__ work");
  FusedCode fc;
  Launch l;
  l.source = std::string(kPrelude) + kernelHeader(leaves, outs) + " {\n" + s.str();
  l.grid[0] = (unsigned)std::max<int64_t>(1, outer * inner);
  l.block[0] = 256;
  for (auto* v : leaves) { KArg a; a.kind = KArg::In; a.value = v; l.args.push_back(a); }
  for (auto& r : sort->results) { KArg a; a.kind = KArg::Out; a.value = r.get(); l.args.push_back(a); }
  if (!inLds) {
    KArg a;
    a.kind = KArg::Work;
    a.workOffset = 0;
    l.args.push_back(a);
    fc.workspaceBytes = outer * inner * P * 4;
  }
  fc.leaves = leaves;
  fc.launches.push_back(std::move(l));
  return fc;
}

// Horizontal batching: independent one-dimensional kernels become the segments of one
// launch.  Every generated kernel is kPrelude + one header + body, and addresses its grid
// through blockIdx.x only, so a segment is that body as a device function of the block index.
bool batchableKernel(const std::string& source) {
  const size_t pre = strlen(kPrelude);
  if (source.compare(0, pre, kPrelude) != 0) return false;
  if (source.find("blockIdx.y", pre) != std::string::npos || source.find("blockIdx.z", pre) != std::string::npos) return false;
  if (source.find("gridDim", pre) != std::string::npos) return false;
  return source.compare(pre, 10, "extern \"C\"") == 0;
}

std::string combineKernels(const std::vector<const std::string*>& sources, const std::vector<unsigned>& gridX) {
  const size_t pre = strlen(kPrelude);
  static const std::string head = "extern \"C\" __global__ void __launch_bounds__(256) k(";
  std::ostringstream segs, params, dispatch;
  size_t argNo = 0;
  unsigned start = 0;
  for (size_t k = 0; k < sources.size(); ++k) {
    const std::string& src = *sources[k];
    if (!batchableKernel(src) || src.compare(pre, head.size(), head) != 0) return "";
    size_t p0 = pre + head.size();
    size_t p1 = src.find(") {\n", p0);
    size_t end = src.rfind('}');
    if (p1 == std::string::npos || end == std::string::npos || end < p1) return "";
    std::string plist = src.substr(p0, p1 - p0);
    std::string body = src.substr(p1 + 4, end - (p1 + 4));
    for (size_t at = body.find("blockIdx.x"); at != std::string::npos; at = body.find("blockIdx.x", at)) body.replace(at, 10, "seg_bx");
    segs << "static __device__ __forceinline__ void seg" << k << "(const unsigned seg_bx" << (plist.empty() ? "" : ", ") << plist << ") {\n" << body << "}\n";
    dispatch << "  if (b < " << (start + gridX[k]) << "u) { seg" << k << "(b - " << start << "u";
    // each parameter is "<type> <name>"; the wrapper renames them a<N> and drops the no-alias promise,
    // which holds inside one segment but not across segments that read the same buffer
    size_t pos = 0;
    while (pos < plist.size()) {
      size_t comma = plist.find(", ", pos);
      std::string one = plist.substr(pos, comma == std::string::npos ? std::string::npos : comma - pos);
      pos = comma == std::string::npos ? plist.size() : comma + 2;
      size_t sp = one.rfind(' ');
      if (sp == std::string::npos) return "";
      std::string type = one.substr(0, sp);
      size_t r = type.find(" __restrict__");
      if (r != std::string::npos) type.erase(r, 13);
      params << (argNo ? ", " : "") << type << " a" << argNo;
      dispatch << ", a" << argNo;
      ++argNo;
    }
    dispatch << "); return; }\n";
    start += gridX[k];
  }
  std::ostringstream s;
  s << kPrelude << segs.str() << head << params.str() << ") {\n  const unsigned b = blockIdx.x;\n" << dispatch.str() << "}\n";
  return s.str();
}

}  // namespace mi355
