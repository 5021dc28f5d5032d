// StableHLO text front end.
//
// Reads the textual MLIR that `jax.jit(f).lower(...).as_text()` prints (pretty
// forms) and the generic `"stablehlo.op"(...) <{...}> ({regions}) : type` form,
// and produces the IR in ir.h with attributes normalised to one spelling per op.
// This replaces the MLIR-library based parser of the reference
// (src/pjrt_plugin/stablehlo_parser.cc:263-285, text fallback at :276-282).
#include <cctype>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <unordered_map>

#include "ir.h"

namespace mi355 {

const char* dtypeName(DType d) {
  switch (d) {
    case DType::Pred: return "i1";
    case DType::S8: return "i8";
    case DType::S16: return "i16";
    case DType::S32: return "i32";
    case DType::S64: return "i64";
    case DType::U8: return "ui8";
    case DType::U16: return "ui16";
    case DType::U32: return "ui32";
    case DType::U64: return "ui64";
    case DType::F16: return "f16";
    case DType::F32: return "f32";
    case DType::F64: return "f64";
    case DType::BF16: return "bf16";
    case DType::Token: return "token";
    default: return "invalid";
  }
}

DType dtypeFromName(const std::string& s) {
  static const std::unordered_map<std::string, DType> m = {
      {"i1", DType::Pred},  {"i8", DType::S8},    {"i16", DType::S16},  {"i32", DType::S32}, {"i64", DType::S64},
      {"ui8", DType::U8},   {"ui16", DType::U16}, {"ui32", DType::U32}, {"ui64", DType::U64}, {"f16", DType::F16},
      {"f32", DType::F32},  {"f64", DType::F64},  {"bf16", DType::BF16}, {"u8", DType::U8},  {"u16", DType::U16},
      {"u32", DType::U32},  {"u64", DType::U64},  {"si32", DType::S32}, {"si64", DType::S64}, {"si8", DType::S8},
      {"si16", DType::S16}, {"index", DType::S64}};
  auto it = m.find(s);
  return it == m.end() ? DType::Invalid : it->second;
}

std::string TensorType::str() const {
  std::string s = "tensor<";
  for (auto d : dims) s += std::to_string(d) + "x";
  s += dtypeName(dt);
  return s + ">";
}

static uint16_t f32ToBf16Bits(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x40);
  u += 0x7FFFu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

static uint16_t f32ToF16Bits(float f) {
  _Float16 h = (_Float16)f;
  uint16_t b;
  memcpy(&b, &h, 2);
  return b;
}

namespace {

struct Scope {
  std::unordered_map<std::string, std::vector<Value*>> names;
};

class Parser {
 public:
  Parser(const char* d, size_t n) : s_(d), n_(n) {}

  std::unique_ptr<Module> parseModule() {
    auto m = std::make_unique<Module>();
    skipAliasLines();
    bool wrapped = false;
    if (eatWord("module")) {
      wrapped = true;
      ws();
      if (peekc() == '@') { ++i_; ident(); }
      if (eatWord("attributes")) moduleAttributes(*m);
      expect("{");
    } else if (peek("builtin.module")) {
      i_ += 14;
      wrapped = true;
      if (eatWord("attributes")) moduleAttributes(*m);
      expect("{");
    }
    skipAliasLines();
    while (true) {
      ws();
      if (i_ >= n_) break;
      if (wrapped && eat("}")) break;
      skipAliasLines();
      if (i_ >= n_) break;
      // Shardy's module-level declarations (sdy.mesh @mesh = <["x"=1]>) say nothing a single device needs: skipped, as
      // the reference lets unregistered dialects pass (stablehlo_parser.cc:74-75)
      if (peek("sdy.")) {
        while (i_ < n_ && s_[i_] != '\n') ++i_;
        continue;
      }
      m->funcs.push_back(parseFunc());
    }
    if (wrapped) skipLoc();
    skipAliasLines();
    if (!m->main()) {
      // a module with a single function is accepted under any name
      if (m->funcs.size() == 1) m->funcs[0]->name = "main";
      else fail("module has no @main function");
    }
    return m;
  }

 private:
  const char* s_;
  size_t n_;
  size_t i_ = 0;
  int nextId_ = 0;
  std::vector<Scope> scopes_;

  // ------------------------------------------------------------ lexing helpers
  [[noreturn]] void fail(const std::string& msg) {
    int line = 1;
    for (size_t k = 0; k < i_ && k < n_; ++k) if (s_[k] == '\n') ++line;
    std::string ctx(s_ + std::min(i_, n_), std::min<size_t>(48, n_ - std::min(i_, n_)));
    for (auto& c : ctx) if (c == '\n') c = ' ';
    throw CompileError("StableHLO parse error at line " + std::to_string(line) + ": " + msg + " near '" + ctx + "'");
  }
  // line of the read position; positions only move forward between calls, so the count resumes where it stopped
  size_t lineScanned_ = 0;
  int lineAtScan_ = 1;
  int currentLine() {
    if (i_ < lineScanned_) { lineScanned_ = 0; lineAtScan_ = 1; }
    for (; lineScanned_ < i_ && lineScanned_ < n_; ++lineScanned_) if (s_[lineScanned_] == '\n') ++lineAtScan_;
    return lineAtScan_;
  }
  void ws() {
    while (i_ < n_) {
      char c = s_[i_];
      if (c == ' ' || c == '\t' || c == '\n' || c == '\r') ++i_;
      else if (c == '/' && i_ + 1 < n_ && s_[i_ + 1] == '/') { while (i_ < n_ && s_[i_] != '\n') ++i_; }
      else break;
    }
  }
  char peekc() { ws(); return i_ < n_ ? s_[i_] : '\0'; }
  bool peek(const char* lit) {
    ws();
    size_t L = strlen(lit);
    return i_ + L <= n_ && memcmp(s_ + i_, lit, L) == 0;
  }
  bool eat(const char* lit) {
    if (!peek(lit)) return false;
    i_ += strlen(lit);
    return true;
  }
  static bool isIdentChar(char c) { return isalnum((unsigned char)c) || c == '_' || c == '.' || c == '$'; }
  bool eatWord(const char* w) {
    ws();
    size_t L = strlen(w);
    if (i_ + L <= n_ && memcmp(s_ + i_, w, L) == 0 && (i_ + L == n_ || !isIdentChar(s_[i_ + L]))) {
      i_ += L;
      return true;
    }
    return false;
  }
  void expect(const char* lit) {
    if (!eat(lit)) fail(std::string("expected '") + lit + "'");
  }
  std::string ident() {
    ws();
    size_t b = i_;
    if (i_ < n_ && (isalpha((unsigned char)s_[i_]) || s_[i_] == '_')) {
      while (i_ < n_ && isIdentChar(s_[i_])) ++i_;
    }
    if (b == i_) fail("identifier expected");
    return std::string(s_ + b, i_ - b);
  }
  // the name after `@`: bare identifier or quoted string
  std::string symbolName() {
    ws();
    if (i_ < n_ && s_[i_] == '"') return stringLit();
    return ident();
  }
  std::string ssaName() {
    ws();
    if (i_ >= n_ || s_[i_] != '%') fail("SSA value expected");
    size_t b = i_++;
    while (i_ < n_ && (isIdentChar(s_[i_]) || s_[i_] == '-')) ++i_;
    if (i_ < n_ && s_[i_] == '#') {
      ++i_;
      while (i_ < n_ && isdigit((unsigned char)s_[i_])) ++i_;
    }
    return std::string(s_ + b, i_ - b);
  }
  std::string stringLit() {
    ws();
    if (i_ >= n_ || s_[i_] != '"') fail("string expected");
    ++i_;
    std::string out;
    while (i_ < n_ && s_[i_] != '"') {
      if (s_[i_] == '\\' && i_ + 1 < n_) {
        char c = s_[i_ + 1];
        if (isxdigit((unsigned char)c) && i_ + 2 < n_ && isxdigit((unsigned char)s_[i_ + 2])) {
          out.push_back((char)strtol(std::string(s_ + i_ + 1, 2).c_str(), nullptr, 16));
          i_ += 3;
          continue;
        }
        out.push_back(c == 'n' ? '\n' : c == 't' ? '\t' : c);
        i_ += 2;
      } else {
        out.push_back(s_[i_++]);
      }
    }
    if (i_ >= n_) fail("unterminated string");
    ++i_;
    return out;
  }
  int64_t integer() {
    ws();
    size_t b = i_;
    if (i_ < n_ && (s_[i_] == '-' || s_[i_] == '+')) ++i_;
    while (i_ < n_ && isdigit((unsigned char)s_[i_])) ++i_;
    if (b == i_ || (i_ == b + 1 && !isdigit((unsigned char)s_[b]))) fail("integer expected");
    return strtoll(std::string(s_ + b, i_ - b).c_str(), nullptr, 10);
  }
  std::vector<int64_t> intList(char open = '[', char close = ']') {
    std::vector<int64_t> out;
    char o[2] = {open, 0}, c[2] = {close, 0};
    expect(o);
    if (eat(c)) return out;
    while (true) {
      out.push_back(integer());
      if (eat(c)) return out;
      expect(",");
    }
  }
  // `loc(...)` after an op, a block argument or a function signature: debug information only
  void skipLoc() {
    size_t save = i_;
    ws();
    if (i_ + 4 <= n_ && memcmp(s_ + i_, "loc(", 4) == 0) {
      i_ += 3;
      skipBalanced('(', ')');
      return;
    }
    i_ = save;
  }
  // `#loc3 = loc("f.py":12:4)` and other `#alias = ...` definitions outside functions: read to the end of the
  // definition (brackets and strings balanced) and dropped, since only locations are ever referred to by alias here
  void skipAliasLines() {
    while (true) {
      ws();
      if (i_ >= n_ || s_[i_] != '#') return;
      int depth = 0;
      while (i_ < n_) {
        char c = s_[i_];
        if (c == '"') { stringLit(); continue; }
        if (c == '(' || c == '[' || c == '{' || c == '<') ++depth;
        else if (c == ')' || c == ']' || c == '}' || c == '>') --depth;
        else if (c == '\n' && depth <= 0) break;
        ++i_;
      }
    }
  }
  // the module's attribute dictionary: only the partition and replica counts matter here
  void moduleAttributes(Module& m) {
    ws();
    const size_t from = i_;
    skipBalanced('{', '}');
    const std::string text(s_ + from, s_ + i_);
    auto count = [&](const char* key, int64_t& out) {
      size_t at = text.find(key);
      if (at == std::string::npos) return;
      at = text.find('=', at);
      if (at == std::string::npos) return;
      out = strtoll(text.c_str() + at + 1, nullptr, 10);
    };
    count("mhlo.num_partitions", m.numPartitions);
    count("mhlo.num_replicas", m.numReplicas);
  }

  void skipBalanced(char open, char close) {
    ws();
    if (i_ >= n_ || s_[i_] != open) fail(std::string("expected '") + open + "'");
    int depth = 0;
    while (i_ < n_) {
      char c = s_[i_];
      if (c == '"') { stringLit(); continue; }
      if (c == open) ++depth;
      else if (c == close) { --depth; if (depth == 0) { ++i_; return; } }
      ++i_;
    }
    fail("unbalanced brackets");
  }

  // ---------------------------------------------------------------- types
  TensorType parseType() {
    ws();
    TensorType t;
    if (eat("tensor<")) {
      while (true) {
        ws();
        if (i_ < n_ && isdigit((unsigned char)s_[i_])) {
          size_t b = i_;
          while (i_ < n_ && isdigit((unsigned char)s_[i_])) ++i_;
          if (i_ < n_ && s_[i_] == 'x') {
            t.dims.push_back(strtoll(std::string(s_ + b, i_ - b).c_str(), nullptr, 10));
            ++i_;
            continue;
          }
          fail("malformed tensor type");
        }
        if (i_ < n_ && s_[i_] == '?') fail("dynamic shapes are not supported");
        break;
      }
      std::string e = ident();
      t.dt = dtypeFromName(e);
      if (t.dt == DType::Invalid) {
        if (e == "complex") fail("complex element types are not supported");
        fail("unsupported element type " + e);
      }
      // optional encoding after a comma
      ws();
      if (i_ < n_ && s_[i_] == ',') { while (i_ < n_ && s_[i_] != '>') ++i_; }
      expect(">");
      return t;
    }
    if (eat("!stablehlo.token") || eat("!mhlo.token")) {
      t.dt = DType::Token;
      return t;
    }
    if (eat("tuple<")) fail("tuple types are not supported");
    std::string e = ident();
    t.dt = dtypeFromName(e);
    if (t.dt == DType::Invalid) fail("unknown type " + e);
    return t;
  }
  std::vector<TensorType> typeListParen() {
    std::vector<TensorType> out;
    expect("(");
    if (eat(")")) return out;
    while (true) {
      out.push_back(parseType());
      if (peekc() == '{') skipBalanced('{', '}');
      if (eat(")")) return out;
      expect(",");
    }
  }
  std::vector<TensorType> typesBare() {
    std::vector<TensorType> out;
    out.push_back(parseType());
    while (eat(",")) out.push_back(parseType());
    return out;
  }

  // ------------------------------------------------------------ attributes
  static void appendElem(std::vector<uint8_t>& out, DType dt, double fv, int64_t iv, uint64_t uv, bool isBits) {
    switch (dt) {
      case DType::F32: { float f = (float)fv; uint32_t u; if (isBits) u = (uint32_t)uv; else memcpy(&u, &f, 4); for (int k = 0; k < 4; ++k) out.push_back((u >> (8 * k)) & 0xFF); break; }
      case DType::F64: { uint64_t u; if (isBits) u = uv; else memcpy(&u, &fv, 8); for (int k = 0; k < 8; ++k) out.push_back((u >> (8 * k)) & 0xFF); break; }
      case DType::BF16: { uint16_t u = isBits ? (uint16_t)uv : f32ToBf16Bits((float)fv); out.push_back(u & 0xFF); out.push_back(u >> 8); break; }
      case DType::F16: { uint16_t u = isBits ? (uint16_t)uv : f32ToF16Bits((float)fv); out.push_back(u & 0xFF); out.push_back(u >> 8); break; }
      case DType::Pred: out.push_back(iv != 0 ? 1 : 0); break;
      default: {
        size_t sz = dtypeSize(dt);
        uint64_t u = (uint64_t)iv;
        for (size_t k = 0; k < sz; ++k) out.push_back((u >> (8 * k)) & 0xFF);
      }
    }
  }

  Attr parseDense() {
    expect("dense<");
    ws();
    struct Tok { bool isBits; bool isFloatText; double f; int64_t i; uint64_t u; };
    std::vector<Tok> toks;
    std::string hex;
    bool isHex = false;
    if (peekc() == '"') {
      hex = stringLit();
      isHex = true;
      expect(">");
    } else {
      int depth = 0;
      while (true) {
        ws();
        if (i_ >= n_) fail("unterminated dense attribute");
        char c = s_[i_];
        if (c == '[') { ++depth; ++i_; continue; }
        if (c == ']') { --depth; ++i_; continue; }
        if (c == ',') { ++i_; continue; }
        if (c == '>' && depth == 0) { ++i_; break; }
        if (c == '(') fail("complex constants are not supported");
        Tok t{false, false, 0, 0, 0};
        if (eatWord("true")) { t.i = 1; t.f = 1; }
        else if (eatWord("false")) { t.i = 0; }
        else {
          size_t b = i_;
          while (i_ < n_ && (isalnum((unsigned char)s_[i_]) || s_[i_] == '.' || s_[i_] == '-' || s_[i_] == '+')) ++i_;
          std::string tk(s_ + b, i_ - b);
          if (tk.empty()) fail("bad dense element");
          if (tk.size() > 2 && tk[0] == '0' && (tk[1] == 'x' || tk[1] == 'X')) {
            t.isBits = true;
            t.u = strtoull(tk.c_str(), nullptr, 16);
            t.i = (int64_t)t.u;
          } else if (tk.find_first_of(".eEn") != std::string::npos && !(tk[0] == '-' && tk.find_first_of(".eEn") == std::string::npos)) {
            t.isFloatText = true;
            t.f = strtod(tk.c_str(), nullptr);
            t.i = (int64_t)t.f;
          } else {
            t.i = strtoll(tk.c_str(), nullptr, 10);
            if (tk[0] != '-' ) t.u = strtoull(tk.c_str(), nullptr, 10), t.i = (int64_t)t.u;
            t.f = (double)t.i;
            if (tk[0] != '-') t.f = (double)t.u;
          }
        }
        toks.push_back(t);
      }
    }
    expect(":");
    TensorType ty = parseType();
    Attr a;
    a.kind = Attr::Dense;
    a.dense = std::make_shared<DenseData>();
    a.dense->type = ty;
    size_t n = (size_t)ty.numel();
    size_t esz = dtypeSize(ty.dt);
    if (isHex) {
      if (hex.size() < 2 || hex[0] != '0' || (hex[1] != 'x' && hex[1] != 'X')) fail("dense string must be a hex blob");
      std::vector<uint8_t> raw;
      raw.reserve((hex.size() - 2) / 2);
      auto hv = [&](char c) -> int { return c <= '9' ? c - '0' : (c | 0x20) - 'a' + 10; };
      for (size_t k = 2; k + 1 < hex.size(); k += 2) raw.push_back((uint8_t)(hv(hex[k]) * 16 + hv(hex[k + 1])));
      if (ty.dt == DType::Pred && raw.size() != n && raw.size() != 1 && raw.size() == (n + 7) / 8) {
        std::vector<uint8_t> un(n);
        for (size_t k = 0; k < n; ++k) un[k] = (raw[k / 8] >> (k % 8)) & 1;
        raw.swap(un);
      }
      if (raw.size() == esz && n != 1) a.dense->splat = true;
      else if (raw.size() != n * esz) fail("dense hex blob has the wrong size");
      a.dense->bytes.swap(raw);
    } else {
      if (toks.size() == 1 && n != 1) a.dense->splat = true;
      else if (toks.size() != n) fail("dense literal has " + std::to_string(toks.size()) + " elements, type wants " + std::to_string(n));
      for (auto& t : toks) {
        bool bits = t.isBits && isFloat(ty.dt);
        appendElem(a.dense->bytes, ty.dt, t.f, t.i, t.u, bits);
      }
    }
    return a;
  }

  Attr parseAttrValue() {
    ws();
    Attr a;
    if (i_ >= n_) fail("attribute expected");
    char c = s_[i_];
    if (c == '"') {
      a.kind = Attr::Str;
      a.s = stringLit();
      if (eat(":")) parseType();
      return a;
    }
    if (c == '[') {
      ++i_;
      a.kind = Attr::List;
      if (eat("]")) { a.kind = Attr::Ints; return a; }
      while (true) {
        a.list.push_back(parseAttrValue());
        if (eat("]")) break;
        expect(",");
      }
      bool allInt = true;
      for (auto& e : a.list) if (e.kind != Attr::Int) allInt = false;
      if (allInt) {
        a.kind = Attr::Ints;
        for (auto& e : a.list) a.ints.push_back(e.i);
        a.list.clear();
      }
      return a;
    }
    if (c == '{') {
      a.kind = Attr::Dict;
      a.dict = parseAttrDict();
      return a;
    }
    if (c == '#') return parseHashAttr();
    if (c == '@') { ++i_; a.kind = Attr::Str; a.s = symbolName(); return a; }
    if (peek("dense<")) return parseDense();
    if (peek("array<")) {
      i_ += 6;
      ident();
      a.kind = Attr::Ints;
      if (eat(">")) return a;
      expect(":");
      while (true) {
        if (eatWord("true")) a.ints.push_back(1);
        else if (eatWord("false")) a.ints.push_back(0);
        else a.ints.push_back(integer());
        if (eat(">")) return a;
        expect(",");
      }
    }
    if (eatWord("true")) { a.kind = Attr::Bool; a.b = true; a.i = 1; return a; }
    if (eatWord("false")) { a.kind = Attr::Bool; a.b = false; return a; }
    if (eatWord("unit")) { a.kind = Attr::Bool; a.b = true; a.i = 1; return a; }
    if (peek("tensor<")) { a.kind = Attr::Type; a.type = parseType(); return a; }
    if (isdigit((unsigned char)c) || c == '-' || c == '+') {
      size_t b = i_;
      ++i_;
      while (i_ < n_ && (isalnum((unsigned char)s_[i_]) || s_[i_] == '.' || ((s_[i_] == '-' || s_[i_] == '+') && (s_[i_ - 1] == 'e' || s_[i_ - 1] == 'E')))) ++i_;
      std::string tk(s_ + b, i_ - b);
      bool hexv = tk.find("0x") != std::string::npos || tk.find("0X") != std::string::npos;
      if (!hexv && tk.find_first_of(".eE") != std::string::npos) {
        a.kind = Attr::Float;
        a.f = strtod(tk.c_str(), nullptr);
      } else {
        a.kind = Attr::Int;
        a.i = hexv ? (int64_t)strtoull(tk.c_str(), nullptr, 16) : strtoll(tk.c_str(), nullptr, 10);
        a.f = (double)a.i;
      }
      // `1 : i64` is a typed literal; in `dim = 0 : (tensor<...>) -> ...` the colon starts the op's type
      size_t save = i_;
      if (eat(":")) {
        ws();
        bool scalarType = false;
        if (i_ < n_ && isalpha((unsigned char)s_[i_])) {
          size_t e = i_;
          while (e < n_ && isIdentChar(s_[e])) ++e;
          scalarType = dtypeFromName(std::string(s_ + i_, e - i_)) != DType::Invalid;
        }
        if (!scalarType) {
          i_ = save;
        } else {
          TensorType t = parseType();
          if (hexv && t.dt == DType::F32) { uint32_t u = (uint32_t)a.i; float f; memcpy(&f, &u, 4); a.kind = Attr::Float; a.f = f; }
          else if (isFloat(t.dt) && a.kind == Attr::Int && !hexv) { a.kind = Attr::Float; }
        }
      }
      return a;
    }
    // bare identifier (enum keyword, type name ...), possibly with <...>
    a.kind = Attr::Str;
    a.s = ident();
    if (peekc() == '<') skipBalanced('<', '>');
    return a;
  }

  Attr parseHashAttr() {
    expect("#");
    std::string name = ident();
    Attr a;
    a.kind = Attr::Dict;
    a.s = name;
    if (!eat("<")) return a;
    if (name == "stablehlo" || name == "mhlo" || name == "chlo") {
      // #stablehlo<precision DEFAULT>, #stablehlo<comparison_direction LT>, ...
      std::string kind = ident();
      Attr v;
      v.kind = Attr::Str;
      if (peekc() != '>') v.s = ident();
      expect(">");
      v.dict["__kind"].kind = Attr::Str;
      v.dict["__kind"].s = kind;
      return v;
    }
    if (name == "stablehlo.conv" || name == "mhlo.conv") {
      a.kind = Attr::Str;
      a.s = "";
      size_t b = i_;
      int depth = 0;
      while (i_ < n_) {
        char c = s_[i_];
        if (c == '<' || c == '[') ++depth;
        else if (c == ']') --depth;
        else if (c == '>') {
          if (i_ > 0 && s_[i_ - 1] == '-') { ++i_; continue; }
          if (depth == 0) break;
          --depth;
        }
        ++i_;
      }
      a.s = std::string(s_ + b, i_ - b);
      expect(">");
      return a;
    }
    if (name.compare(0, 4, "sdy.") == 0) {
      // Shardy attributes (#sdy.sharding<@mesh, [{}, {"x"}]>): kept as their text, read by nothing
      a.kind = Attr::Str;
      size_t b = i_;
      int depth = 0;
      bool quoted = false;
      for (; i_ < n_; ++i_) {
        char c = s_[i_];
        if (c == '"') quoted = !quoted;
        if (quoted) continue;
        if (c == '<' || c == '[' || c == '{') ++depth;
        else if (c == ']' || c == '}') --depth;
        else if (c == '>') { if (depth == 0) break; --depth; }
      }
      a.s = std::string(s_ + b, i_ - b);
      expect(">");
      return a;
    }
    while (!eat(">")) {
      std::string k = ident();
      expect("=");
      a.dict[k] = parseAttrValue();
      eat(",");
    }
    return a;
  }

  std::map<std::string, Attr> parseAttrDict() {
    std::map<std::string, Attr> d;
    expect("{");
    if (eat("}")) return d;
    while (true) {
      ws();
      std::string k = (i_ < n_ && s_[i_] == '"') ? stringLit() : ident();
      if (eat("=")) d[k] = parseAttrValue();
      else { d[k].kind = Attr::Bool; d[k].b = true; d[k].i = 1; }
      if (eat("}")) return d;
      expect(",");
    }
  }

  // ------------------------------------------------------------- symbols
  void define(const std::string& name, std::vector<Value*> vals) { scopes_.back().names[name] = std::move(vals); }
  Value* lookup(const std::string& full) {
    std::string base = full;
    int idx = -1;
    auto h = full.find('#');
    if (h != std::string::npos) {
      base = full.substr(0, h);
      idx = atoi(full.c_str() + h + 1);
    }
    for (int k = (int)scopes_.size() - 1; k >= 0; --k) {
      auto it = scopes_[k].names.find(base);
      if (it == scopes_[k].names.end()) continue;
      auto& v = it->second;
      if (idx < 0) {
        if (v.size() != 1) fail("value " + full + " has " + std::to_string(v.size()) + " results; use #n");
        return v[0];
      }
      if (idx >= (int)v.size()) fail("result index out of range in " + full);
      return v[idx];
    }
    fail("use of undefined value " + full);
  }
  std::vector<Value*> ssaUseList() {
    std::vector<Value*> out;
    out.push_back(lookup(ssaName()));
    while (true) {
      size_t save = i_;
      if (!eat(",")) break;
      if (peekc() != '%') { i_ = save; break; }
      out.push_back(lookup(ssaName()));
    }
    return out;
  }
  std::unique_ptr<Value> newValue(const TensorType& t, const std::string& name) {
    auto v = std::make_unique<Value>();
    v->id = nextId_++;
    v->type = t;
    v->name = name;
    return v;
  }

  // ----------------------------------------------------------- functions
  std::unique_ptr<Func> parseFunc() {
    if (!eat("func.func")) fail("expected func.func");
    auto f = std::make_unique<Func>();
    if (eatWord("public")) f->isPublic = true;
    else if (eatWord("private")) f->isPublic = false;
    else f->isPublic = true;
    expect("@");
    f->name = symbolName();
    scopes_.emplace_back();
    expect("(");
    if (!eat(")")) {
      while (true) {
        std::string nm = ssaName();
        expect(":");
        auto v = newValue(parseType(), nm);
        v->argOf = &f->body;
        v->defIndex = (int)f->body.args.size();
        define(nm, {v.get()});
        f->body.args.push_back(std::move(v));
        int donation = -1;
        if (peekc() == '{') {
          auto attrs = parseAttrDict();
          auto al = attrs.find("tf.aliasing_output");
          if (al != attrs.end() && al->second.kind == Attr::Int) donation = (int)al->second.i;
          auto dn = attrs.find("jax.buffer_donor");
          if (donation < 0 && dn != attrs.end() && dn->second.b) donation = -2;
        }
        f->argDonation.push_back(donation);
        skipLoc();
        if (eat(")")) break;
        expect(",");
      }
    }
    if (eat("->")) {
      if (peekc() == '(') f->resultTypes = typeListParen();
      else f->resultTypes.push_back(parseType());   // attributes on results need the parenthesised form
    }
    if (eatWord("attributes")) skipBalanced('{', '}');
    expect("{");
    parseBlockOps(f->body);
    expect("}");
    skipLoc();
    scopes_.pop_back();
    return f;
  }

  void parseBlockOps(Region& r) {
    while (true) {
      ws();
      if (peekc() == '}') break;
      if (i_ >= n_) fail("unexpected end of input inside a region");
      auto op = parseOp();
      op->parent = &r;
      r.ops.push_back(std::move(op));
    }
    if (r.ops.empty() || r.ops.back()->name != "return") {
      auto t = std::make_unique<Op>();
      t->name = "return";
      t->parent = &r;
      r.ops.push_back(std::move(t));
    }
  }

  // region with optional ^bb0(args) header; `preArgs` are names already bound by the op syntax
  std::unique_ptr<Region> parseRegion(Op* parent, const std::vector<std::pair<std::string, TensorType>>* preArgs = nullptr) {
    auto r = std::make_unique<Region>();
    r->parent = parent;
    scopes_.emplace_back();
    expect("{");
    if (preArgs) {
      for (auto& p : *preArgs) {
        auto v = newValue(p.second, p.first);
        v->argOf = r.get();
        v->defIndex = (int)r->args.size();
        define(p.first, {v.get()});
        r->args.push_back(std::move(v));
      }
    }
    ws();
    if (peekc() == '^') {
      ++i_;
      ident();
      if (eat("(")) {
        if (!eat(")")) {
          while (true) {
            std::string nm = ssaName();
            expect(":");
            auto v = newValue(parseType(), nm);
            v->argOf = r.get();
            v->defIndex = (int)r->args.size();
            define(nm, {v.get()});
            r->args.push_back(std::move(v));
            skipLoc();
            if (eat(")")) break;
            expect(",");
          }
        }
      }
      expect(":");
    }
    parseBlockOps(*r);
    expect("}");
    scopes_.pop_back();
    return r;
  }

  void setResults(Op* op, const std::vector<TensorType>& types, const std::string& base, int declared) {
    if (declared >= 0 && declared != (int)types.size() && !(declared == 1 && types.size() == 1))
      if (!(declared == 0 && types.empty())) fail("op " + op->name + " declares " + std::to_string(declared) + " results but its type has " + std::to_string(types.size()));
    std::vector<Value*> vals;
    for (size_t k = 0; k < types.size(); ++k) {
      auto v = newValue(types[k], types.size() == 1 ? base : base + "#" + std::to_string(k));
      v->def = op;
      v->defIndex = (int)k;
      vals.push_back(v.get());
      op->results.push_back(std::move(v));
    }
    if (!base.empty()) define(base, vals);
  }

  void fnType(Op* op, std::vector<TensorType>& outs) {
    if (peekc() == '(') {
      typeListParen();
      expect("->");
      if (peekc() == '(') outs = typeListParen();
      else outs.push_back(parseType());
    } else {
      outs.push_back(parseType());
      // chlo's pretty form: `chlo.erf %x : tensor<4xf32> -> tensor<4xf32>`
      if (eat("->")) {
        outs.clear();
        if (peekc() == '(') outs = typeListParen();
        else outs.push_back(parseType());
      }
    }
  }

  std::unique_ptr<Op> parseOp() {
    auto op = std::make_unique<Op>();
    op->line = currentLine();
    ws();
    std::string base;
    int declared = 0;
    // `%a = op`, `%a:2 = op` or `%a, %b = op` (each name stands for `count` consecutive results)
    std::vector<std::pair<std::string, int>> resultNames;
    if (peekc() == '%') {
      while (true) {
        ws();
        if (i_ >= n_ || s_[i_] != '%') fail("result name expected");
        size_t b = i_++;
        while (i_ < n_ && (isIdentChar(s_[i_]) || s_[i_] == '-')) ++i_;
        std::string nm(s_ + b, i_ - b);
        int cnt = 1;
        if (eat(":")) cnt = (int)integer();
        resultNames.emplace_back(nm, cnt);
        declared += cnt;
        if (!eat(",")) break;
      }
      base = resultNames[0].first;
      expect("=");
    }
    ws();
    std::vector<TensorType> outs;
    if (peekc() == '"') {
      std::string full = stringLit();
      op->name = stripDialect(full);
      parseGenericOp(op.get(), outs);
      normalizeGenericAttrs(op.get());
    } else {
      std::string full = ident();
      op->name = stripDialect(full);
      if (op->name == "return") {
        if (peekc() == '%') {
          op->operands = ssaUseList();
          expect(":");
          typesBare();
        }
      } else if (op->name == "call") {
        expect("@");
        op->attrs["callee"].kind = Attr::Str;
        op->attrs["callee"].s = symbolName();
        expect("(");
        if (peekc() != ')') op->operands = ssaUseList();
        expect(")");
        if (peekc() == '{') skipBalanced('{', '}');
        expect(":");
        typeListParen();
        expect("->");
        if (peekc() == '(') outs = typeListParen();
        else outs.push_back(parseType());
      } else {
        parsePrettyOp(op.get(), outs);
      }
    }
    setResults(op.get(), outs, resultNames.size() > 1 ? std::string() : base, base.empty() ? -1 : declared);
    if (resultNames.size() > 1) {
      size_t at = 0;
      for (auto& rn : resultNames) {
        std::vector<Value*> vals;
        for (int k = 0; k < rn.second && at < op->results.size(); ++k) vals.push_back(op->results[at++].get());
        define(rn.first, vals);
      }
    }
    skipLoc();
    return op;
  }

  static std::string stripDialect(const std::string& full) {
    if (full.rfind("stablehlo.", 0) == 0) return full.substr(10);
    if (full.rfind("mhlo.", 0) == 0) return full.substr(5);
    if (full.rfind("func.", 0) == 0) return full.substr(5);
    return full;  // chlo.* and unknown dialects keep their prefix
  }

  void parseGenericOp(Op* op, std::vector<TensorType>& outs) {
    expect("(");
    if (peekc() != ')') op->operands = ssaUseList();
    expect(")");
    if (eat("<")) {
      auto d = parseAttrDict();
      for (auto& kv : d) op->attrs[kv.first] = kv.second;
      expect(">");
    }
    if (peekc() == '(') {
      expect("(");
      while (true) {
        op->regions.push_back(parseRegion(op));
        if (!eat(",")) break;
      }
      expect(")");
    }
    if (peekc() == '{') {
      auto d = parseAttrDict();
      for (auto& kv : d) op->attrs[kv.first] = kv.second;
    }
    expect(":");
    typeListParen();
    expect("->");
    if (peekc() == '(') outs = typeListParen();
    else outs.push_back(parseType());
  }

  static void setInts(Op* op, const std::string& k, const std::vector<int64_t>& v) {
    Attr a;
    a.kind = Attr::Ints;
    a.ints = v;
    op->attrs[k] = a;
  }
  static void setInt(Op* op, const std::string& k, int64_t v) {
    Attr a;
    a.kind = Attr::Int;
    a.i = v;
    op->attrs[k] = a;
  }
  static void setStr(Op* op, const std::string& k, const std::string& v) {
    Attr a;
    a.kind = Attr::Str;
    a.s = v;
    op->attrs[k] = a;
  }
  static std::vector<int64_t> denseToInts(const Attr& a) {
    std::vector<int64_t> out;
    if (a.kind == Attr::Ints) return a.ints;
    if (a.kind != Attr::Dense) return out;
    auto& d = *a.dense;
    size_t esz = dtypeSize(d.type.dt);
    size_t n = (size_t)d.type.numel();
    for (size_t k = 0; k < n; ++k) {
      const uint8_t* p = d.bytes.data() + (d.splat ? 0 : k * esz);
      int64_t v = 0;
      memcpy(&v, p, esz);
      if (esz < 8 && isSignedInt(d.type.dt) && (v >> (8 * esz - 1)) & 1) v |= ~((int64_t(1) << (8 * esz)) - 1);
      out.push_back(v);
    }
    return out;
  }

  void rename(Op* op, const char* from, const char* to) {
    auto it = op->attrs.find(from);
    if (it == op->attrs.end()) return;
    Attr a = it->second;
    if (a.kind == Attr::Dense) { Attr b; b.kind = Attr::Ints; b.ints = denseToInts(a); a = b; }
    op->attrs.erase(it);
    op->attrs[to] = a;
  }

  void parseConvSpec(const std::string& spec, ConvDims& cd) {
    // "[b, 0, 1, f]x[0, 1, i, o]->[b, 0, 1, f]"
    std::vector<std::vector<std::string>> parts;
    size_t k = 0;
    while (k < spec.size()) {
      if (spec[k] == '[') {
        parts.emplace_back();
        ++k;
        std::string cur;
        while (k < spec.size() && spec[k] != ']') {
          if (spec[k] == ',') { parts.back().push_back(cur); cur.clear(); }
          else if (!isspace((unsigned char)spec[k])) cur.push_back(spec[k]);
          ++k;
        }
        if (!cur.empty()) parts.back().push_back(cur);
      }
      ++k;
    }
    if (parts.size() != 3) fail("malformed convolution dimension numbers");
    int nsp = (int)parts[0].size() - 2;
    if (nsp < 0) fail("convolution needs at least batch and feature dims");
    cd.lhsSpatial.assign(nsp, -1);
    cd.rhsSpatial.assign(nsp, -1);
    cd.outSpatial.assign(nsp, -1);
    for (int d = 0; d < (int)parts[0].size(); ++d) {
      auto& t = parts[0][d];
      if (t == "b") cd.lhsBatch = d; else if (t == "f") cd.lhsFeature = d; else cd.lhsSpatial.at(atoi(t.c_str())) = d;
    }
    for (int d = 0; d < (int)parts[1].size(); ++d) {
      auto& t = parts[1][d];
      if (t == "i") cd.rhsIn = d; else if (t == "o") cd.rhsOut = d; else cd.rhsSpatial.at(atoi(t.c_str())) = d;
    }
    for (int d = 0; d < (int)parts[2].size(); ++d) {
      auto& t = parts[2][d];
      if (t == "b") cd.outBatch = d; else if (t == "f") cd.outFeature = d; else cd.outSpatial.at(atoi(t.c_str())) = d;
    }
  }

  // Generic-form attribute names -> the names the pretty forms use.
  void normalizeGenericAttrs(Op* op) {
    const std::string& n = op->name;
    if (n == "broadcast_in_dim") rename(op, "broadcast_dimensions", "dims");
    else if (n == "transpose") rename(op, "permutation", "dims");
    else if (n == "reverse") rename(op, "dimensions", "dims");
    else if (n == "concatenate") rename(op, "dimension", "dim");
    else if (n == "iota") rename(op, "iota_dimension", "dim");
    else if (n == "reduce") rename(op, "dimensions", "dimensions");
    else if (n == "slice") { rename(op, "start_indices", "start"); rename(op, "limit_indices", "limit"); rename(op, "strides", "strides"); }
    else if (n == "dynamic_slice") rename(op, "slice_sizes", "sizes");
    else if (n == "pad") { rename(op, "edge_padding_low", "low"); rename(op, "edge_padding_high", "high"); rename(op, "interior_padding", "interior"); }
    else if (n == "compare") {
      auto it = op->attrs.find("comparison_direction");
      if (it != op->attrs.end()) { setStr(op, "direction", it->second.s); op->attrs.erase("comparison_direction"); }
      it = op->attrs.find("compare_type");
      if (it != op->attrs.end()) { std::string s = it->second.s; op->attrs.erase("compare_type"); setStr(op, "compare_type", s); }
    } else if (n == "constant") {
      // "value" stays
    } else if (n == "dot_general") {
      auto it = op->attrs.find("dot_dimension_numbers");
      if (it != op->attrs.end()) {
        auto& d = it->second.dict;
        setInts(op, "lhs_batch", d.count("lhs_batching_dimensions") ? d["lhs_batching_dimensions"].ints : std::vector<int64_t>{});
        setInts(op, "rhs_batch", d.count("rhs_batching_dimensions") ? d["rhs_batching_dimensions"].ints : std::vector<int64_t>{});
        setInts(op, "lhs_contract", d.count("lhs_contracting_dimensions") ? d["lhs_contracting_dimensions"].ints : std::vector<int64_t>{});
        setInts(op, "rhs_contract", d.count("rhs_contracting_dimensions") ? d["rhs_contracting_dimensions"].ints : std::vector<int64_t>{});
        op->attrs.erase("dot_dimension_numbers");
      }
    } else if (n == "dot") {
      // plain dot: contract last of lhs with first of rhs
    } else if (n == "gather" || n == "scatter") {
      const char* key = n == "gather" ? "dimension_numbers" : "scatter_dimension_numbers";
      auto it = op->attrs.find(key);
      if (it != op->attrs.end()) {
        auto d = it->second.dict;
        for (auto& kv : d) {
          if (kv.second.kind == Attr::Ints) setInts(op, kv.first, kv.second.ints);
          else if (kv.second.kind == Attr::Int) setInt(op, kv.first, kv.second.i);
        }
        op->attrs.erase(key);
      }
      if (n == "gather") rename(op, "slice_sizes", "slice_sizes");
    } else if (n == "convolution") {
      auto it = op->attrs.find("dimension_numbers");
      if (it != op->attrs.end()) { parseConvSpec(it->second.s, op->convDims); op->attrs.erase("dimension_numbers"); }
      rename(op, "window_strides", "stride");
      rename(op, "lhs_dilation", "lhs_dilate");
      rename(op, "rhs_dilation", "rhs_dilate");
      rename(op, "window_reversal", "reverse");
      rename(op, "padding", "pad");
    } else if (n == "custom_call") {
      auto it = op->attrs.find("call_target_name");
      if (it != op->attrs.end()) setStr(op, "target", it->second.s);
    }
  }

  void parsePrettyOp(Op* op, std::vector<TensorType>& outs) {
    const std::string& n = op->name;
    if (n == "constant") {
      if (peekc() == '{') skipBalanced('{', '}');
      Attr a = parseDense();
      outs.push_back(a.dense->type);
      op->attrs["value"] = a;
      return;
    }
    if (n == "iota") {
      expect("dim");
      expect("=");
      setInt(op, "dim", integer());
      expect(":");
      outs.push_back(parseType());
      return;
    }
    if (n == "compare") {
      setStr(op, "direction", ident());
      expect(",");
      op->operands.push_back(lookup(ssaName()));
      expect(",");
      op->operands.push_back(lookup(ssaName()));
      if (eat(",")) setStr(op, "compare_type", ident());
      expect(":");
      fnType(op, outs);
      return;
    }
    if (n == "reduce") return parseReduce(op, outs);
    if (n == "while") return parseWhile(op, outs);
    if (n == "convolution") return parseConvolution(op, outs);
    if (n == "custom_call") {
      expect("@");
      setStr(op, "target", ident());
      expect("(");
      if (peekc() != ')') op->operands = ssaUseList();
      expect(")");
      if (peekc() == '{') {
        auto d = parseAttrDict();
        for (auto& kv : d) op->attrs[kv.first] = kv.second;
      }
      expect(":");
      fnType(op, outs);
      return;
    }
    if (n == "chlo.top_k") {
      // %values, %indices = chlo.top_k(%x, k = 3) : tensor<16xf32> -> (tensor<3xf32>, tensor<3xi32>)
      expect("(");
      op->operands = ssaUseList();
      expect(",");
      expect("k");
      expect("=");
      setInt(op, "k", integer());
      expect(")");
      if (peekc() == '{') skipBalanced('{', '}');
      expect(":");
      parseType();
      expect("->");
      outs = typeListParen();
      return;
    }
    if (n == "rng_bit_generator") {
      // %state, %bits = stablehlo.rng_bit_generator %state0, algorithm = THREE_FRY : (tensor<2xui64>) -> (tensor<2xui64>, tensor<8xui32>)
      op->operands = ssaUseList();
      expect(",");
      expect("algorithm");
      expect("=");
      setStr(op, "rng_algorithm", ident());
      if (peekc() == '{') skipBalanced('{', '}');
      expect(":");
      fnType(op, outs);
      return;
    }
    if (n == "optimization_barrier") {
      if (peekc() == '%') op->operands = ssaUseList();
      expect(":");
      outs = typesBare();
      return;
    }
    if (n == "composite") {
      // %0 = stablehlo.composite "chlo.asin" %x {decomposition = @chlo.asin.impl} : (tensor<4xf32>) -> tensor<4xf32>
      setStr(op, "name", stringLit());
      if (peekc() == '%') op->operands = ssaUseList();
      if (peekc() == '{') {
        auto d = parseAttrDict();
        for (auto& kv : d) op->attrs[kv.first] = kv.second;
      }
      expect(":");
      fnType(op, outs);
      if (!op->has("decomposition")) fail("stablehlo.composite without a decomposition function");
      return;
    }
    if (n == "reduce_precision") {
      // %0 = stablehlo.reduce_precision %x, format = e5m10 : tensor<16xf32>
      op->operands = ssaUseList();
      expect(",");
      expect("format");
      expect("=");
      ws();
      if (i_ >= n_ || s_[i_] != 'e') fail("expected a format of the form e<exponent bits>m<mantissa bits>");
      ++i_;
      setInt(op, "exponent_bits", integer());
      if (i_ >= n_ || s_[i_] != 'm') fail("expected a format of the form e<exponent bits>m<mantissa bits>");
      ++i_;
      setInt(op, "mantissa_bits", integer());
      if (peekc() == '{') skipBalanced('{', '}');
      expect(":");
      fnType(op, outs);
      return;
    }
    // common pretty form: operands, keyword attributes, optional attr dict, type
    if (peekc() == '%') op->operands = ssaUseList();
    if (n == "slice") {
      std::vector<int64_t> st, li, sr;
      expect("[");
      if (!eat("]")) {
        while (true) {
          st.push_back(integer());
          expect(":");
          li.push_back(integer());
          sr.push_back(eat(":") ? integer() : 1);
          if (eat("]")) break;
          expect(",");
        }
      }
      setInts(op, "start", st);
      setInts(op, "limit", li);
      setInts(op, "strides", sr);
    }
    while (eat(",")) {
      std::string k = ident();
      expect("=");
      if (k == "batching_dims" || k == "contracting_dims") {
        auto a = intList();
        expect("x");
        auto b = intList();
        setInts(op, k == "batching_dims" ? "lhs_batch" : "lhs_contract", a);
        setInts(op, k == "batching_dims" ? "rhs_batch" : "rhs_contract", b);
      } else {
        op->attrs[k] = parseAttrValue();
      }
    }
    if (peekc() == '{') {
      auto d = parseAttrDict();
      for (auto& kv : d) op->attrs[kv.first] = kv.second;
    }
    expect(":");
    if (n == "select" && peekc() != '(') {
      parseType();
      expect(",");
      outs.push_back(parseType());
    } else {
      fnType(op, outs);
    }
    if (n == "dot_general") {
      for (const char* k : {"lhs_batch", "rhs_batch", "lhs_contract", "rhs_contract"})
        if (!op->has(k)) setInts(op, k, {});
    }
    normalizeGenericAttrs(op);  // tolerates generic names inside a trailing attr dict
  }

  void parseReduce(Op* op, std::vector<TensorType>& outs) {
    std::vector<Value*> ins, inits;
    while (true) {
      expect("(");
      ins.push_back(lookup(ssaName()));
      expect("init:");
      inits.push_back(lookup(ssaName()));
      expect(")");
      if (!eat(",")) break;
    }
    op->operands = ins;
    op->operands.insert(op->operands.end(), inits.begin(), inits.end());
    std::string applies;
    if (eatWord("applies")) applies = stripDialect(ident());
    expect("across");
    expect("dimensions");
    expect("=");
    setInts(op, "dimensions", intList());
    if (peekc() == '{') skipBalanced('{', '}');
    expect(":");
    fnType(op, outs);
    if (!applies.empty()) {
      auto r = std::make_unique<Region>();
      r->parent = op;
      TensorType st;
      st.dt = outs.at(0).dt;
      for (int k = 0; k < 2; ++k) {
        auto v = newValue(st, k == 0 ? "%lhs" : "%rhs");
        v->argOf = r.get();
        v->defIndex = k;
        r->args.push_back(std::move(v));
      }
      auto body = std::make_unique<Op>();
      body->name = applies;
      body->parent = r.get();
      body->operands = {r->args[0].get(), r->args[1].get()};
      auto res = newValue(st, "%red");
      res->def = body.get();
      body->results.push_back(std::move(res));
      auto ret = std::make_unique<Op>();
      ret->name = "return";
      ret->parent = r.get();
      ret->operands = {body->results[0].get()};
      r->ops.push_back(std::move(body));
      r->ops.push_back(std::move(ret));
      op->regions.push_back(std::move(r));
      return;
    }
    if (!eatWord("reducer")) fail("expected 'reducer' region on stablehlo.reduce");
    std::vector<std::pair<std::string, TensorType>> lhs, rhs;
    while (eat("(")) {
      std::string a = ssaName();
      expect(":");
      TensorType ta = parseType();
      expect(",");
      std::string b = ssaName();
      expect(":");
      TensorType tb = parseType();
      expect(")");
      lhs.emplace_back(a, ta);
      rhs.emplace_back(b, tb);
    }
    lhs.insert(lhs.end(), rhs.begin(), rhs.end());
    op->regions.push_back(parseRegion(op, &lhs));
  }

  void parseWhile(Op* op, std::vector<TensorType>& outs) {
    std::vector<std::string> names;
    expect("(");
    if (!eat(")")) {
      while (true) {
        names.push_back(ssaName());
        expect("=");
        op->operands.push_back(lookup(ssaName()));
        if (eat(")")) break;
        expect(",");
      }
    }
    if (eat(":")) outs = typesBare();
    if (outs.size() != names.size()) fail("while: iteration argument / type count mismatch");
    if (eatWord("attributes")) skipBalanced('{', '}');
    std::vector<std::pair<std::string, TensorType>> pre;
    for (size_t k = 0; k < names.size(); ++k) pre.emplace_back(names[k], outs[k]);
    if (!eatWord("cond")) fail("expected 'cond'");
    op->regions.push_back(parseRegion(op, &pre));
    if (!eatWord("do")) fail("expected 'do'");
    op->regions.push_back(parseRegion(op, &pre));
  }

  void parseConvolution(Op* op, std::vector<TensorType>& outs) {
    expect("(");
    op->operands = ssaUseList();
    expect(")");
    expect("dim_numbers");
    expect("=");
    ws();
    size_t b = i_;
    // up to the comma that follows the third bracket group
    int groups = 0;
    while (i_ < n_ && groups < 3) {
      if (s_[i_] == ']') ++groups;
      ++i_;
    }
    parseConvSpec(std::string(s_ + b, i_ - b), op->convDims);
    expect(",");
    expect("window");
    expect("=");
    expect("{");
    while (!eat("}")) {
      std::string k = ident();
      expect("=");
      Attr a = parseAttrValue();
      if (k == "pad") {
        Attr p;
        p.kind = Attr::Ints;
        for (auto& row : a.list) for (auto v : row.ints) p.ints.push_back(v);
        if (a.kind == Attr::Ints) p.ints = a.ints;
        op->attrs["pad"] = p;
      } else if (k == "reverse") {
        Attr p;
        p.kind = Attr::Ints;
        for (auto& e : a.list) p.ints.push_back(e.b ? 1 : 0);
        if (a.kind == Attr::Ints) p.ints = a.ints;
        op->attrs["reverse"] = p;
      } else {
        op->attrs[k] = a;
      }
      eat(",");
    }
    if (peekc() == '{') {
      auto d = parseAttrDict();
      for (auto& kv : d) op->attrs[kv.first] = kv.second;
    }
    expect(":");
    fnType(op, outs);
  }
};

}  // namespace

std::unique_ptr<Module> parseStableHLOText(const char* data, size_t size) {
  if (isMlirBytecode(data, size)) {
    // what jaxlib sends: a VHLO portable artifact in MLIR bytecode (reference: stablehlo_parser.cc:263-285)
    std::string text = vhloBytecodeToStableHLOText(data, size);
    if (getenv("MI355X_DUMP_BYTECODE_TEXT")) fprintf(stderr, "%s\n", text.c_str());
    Parser p(text.data(), text.size());
    return p.parseModule();
  }
  Parser p(data, size);
  return p.parseModule();
}

}  // namespace mi355
