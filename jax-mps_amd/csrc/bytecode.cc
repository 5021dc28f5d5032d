// MLIR bytecode front end: reads a VHLO portable artifact (what jaxlib hands PJRT_Client_Compile) and rewrites it as
// StableHLO text in the generic op form, which parser.cc then reads.  This replaces the deserialisation the reference
// gets from the MLIR / StableHLO libraries (src/pjrt_plugin/stablehlo_parser.cc:263-285: deserializePortableArtifact
// first, text second).
//
// Container format (MLIR bytecode, versions 0 - 6): magic "ML\xEFR", version (varint), producer string, then sections
// {id | aligned << 7, length, [alignment, 0xCB padding], data} for strings (0), dialects and op names (1), attribute /
// type data (2) and offsets (3), IR (4), resources (5, 6), properties (8).  Attributes and types are decoded on demand.
// The builtin dialect's dictionary / string attributes and the vhlo dialect's attribute and type encodings are the ones
// a portable artifact uses; the code tables below restate those dialects' encodings.  No artifact written by jaxlib
// is available offline, so the tables are checked only against this repository's own writer (tests/vhlo_writer.py).
#include <cstdint>
#include <cstring>
#include <map>
#include <sstream>
#include <string>
#include <vector>

#include "ir.h"

namespace mi355 {

namespace {

[[noreturn]] void bad(const std::string& msg) { throw CompileError("MLIR bytecode: " + msg); }

struct Cursor {
  const uint8_t* base = nullptr;   // start of the whole file (alignment is relative to it)
  const uint8_t* p = nullptr;
  const uint8_t* end = nullptr;
  bool empty() const { return p >= end; }
  size_t left() const { return (size_t)(end - p); }
  uint8_t byte() {
    if (p >= end) bad("unexpected end of data");
    return *p++;
  }
  // Prefix varint: the number of trailing zero bits of the first byte is the number of bytes that follow.
  uint64_t varint() {
    uint8_t first = byte();
    if (first & 1) return first >> 1;
    if (first == 0) {
      if (left() < 8) bad("truncated varint");
      uint64_t v;
      memcpy(&v, p, 8);
      p += 8;
      return v;
    }
    int extra = __builtin_ctz((unsigned)first);
    if ((int)left() < extra) bad("truncated varint");
    uint64_t v = first;
    for (int k = 0; k < extra; ++k) v |= (uint64_t)p[k] << (8 * (k + 1));
    p += extra;
    return v >> (extra + 1);
  }
  int64_t svarint() {
    uint64_t v = varint();
    return (int64_t)(v >> 1) ^ -(int64_t)(v & 1);
  }
  uint64_t varintFlag(bool& flag) {
    uint64_t v = varint();
    flag = (v & 1) != 0;
    return v >> 1;
  }
  Cursor take(size_t n) {
    if (left() < n) bad("section or blob runs past the end of the data");
    Cursor c;
    c.base = base;
    c.p = p;
    c.end = p + n;
    p += n;
    return c;
  }
  void alignTo(uint64_t alignment) {
    if (alignment == 0 || (alignment & (alignment - 1))) bad("alignment is not a power of two");
    while (((uint64_t)(p - base) & (alignment - 1)) != 0) {
      if (byte() != 0xCB) bad("bad alignment padding");
    }
  }
  std::string cstring() {
    const uint8_t* s = p;
    while (p < end && *p) ++p;
    if (p >= end) bad("unterminated string");
    std::string out((const char*)s, (size_t)(p - s));
    ++p;
    return out;
  }
};

enum SectionId { kString = 0, kDialect = 1, kAttrType = 2, kAttrTypeOffset = 3, kIR = 4, kResource = 5, kResourceOffset = 6, kDialectVersions = 7, kProperties = 8 };

// one section header at the cursor; returns its id and payload
int readSection(Cursor& c, Cursor& payload) {
  uint8_t idByte = c.byte();
  int id = idByte & 0x7F;
  bool aligned = (idByte & 0x80) != 0;
  uint64_t length = c.varint();
  if (aligned) c.alignTo(c.varint());
  payload = c.take((size_t)length);
  return id;
}

// ---- code tables ---------------------------------------------------------------------------------------------------
// builtin dialect attribute codes used by a portable artifact's op attribute dictionaries
enum BuiltinAttrCode { kBuiltinArrayAttr = 0, kBuiltinDictionaryAttr = 1, kBuiltinStringAttr = 2, kBuiltinStringAttrWithType = 3,
                       kBuiltinFlatSymbolRefAttr = 4, kBuiltinTypeAttr = 6, kBuiltinUnitAttr = 7, kBuiltinIntegerAttr = 8 };
// vhlo attribute codes
enum VhloAttrCode { kArrayV1 = 0, kBooleanV1 = 1, kComparisonDirectionV1 = 2, kComparisonTypeV1 = 3, kCustomCallApiVersionV1 = 4,
                    kDictionaryV1 = 5, kFftTypeV1 = 6, kFloatV1 = 7, kIntegerV1 = 8, kOutputOperandAliasV1 = 9, kPrecisionV1 = 10,
                    kRngAlgorithmV1 = 11, kRngDistributionV1 = 12, kStringV1 = 13, kTensorV1 = 14, kTransposeV1 = 15, kTypeV1 = 16,
                    kTypeExtensionsV1 = 17, kResultAccuracyModeV1 = 18, kResultAccuracyV1 = 19 };
// vhlo type codes
enum VhloTypeCode { kBooleanT = 0, kComplexT = 1, kBF16T = 2, kF16T = 3, kF32T = 4, kF64T = 5, kF8E4M3FNT = 6, kF8E5M2T = 7, kFunctionT = 8,
                    kIndexT = 9, kSI4T = 10, kSI8T = 11, kSI16T = 12, kSI32T = 13, kSI64T = 14, kUI4T = 15, kUI8T = 16, kUI16T = 17,
                    kUI32T = 18, kUI64T = 19, kRankedTensorT = 20, kRankedTensorEncT = 21, kTokenT = 22, kTupleT = 23, kUniformQuantizedT = 24,
                    kUnrankedTensorT = 25, kWitnessT = 26 };

struct BType {
  bool decoded = false;
  bool vhlo = false;
  int code = -1;
  std::vector<int64_t> shape;
  int elem = -1;                  // element type index (tensors, complex)
  std::vector<int> ins, outs;     // function / tuple types
  std::string text;               // printed form
};

struct BAttr {
  bool decoded = false;
  enum Kind { Unknown, Array, Bool, Enum, Dict, Float, Int, String, Tensor, Type, Ints, Symbol, Unit } kind = Unknown;
  std::vector<int> elems;                     // Array: attribute indices
  std::vector<std::pair<int, int>> pairs;     // Dict: (name attribute, value attribute)
  bool b = false;
  int64_t i = 0;
  uint64_t bits = 0;                          // Float: bit pattern
  std::string s, enumKind;
  int type = -1;                              // Int / Float / Tensor / Type: type index
  std::vector<uint8_t> blob;                  // Tensor: raw element data
  std::vector<int64_t> ints;                  // TypeExtensions bounds
  std::string origin;                         // Unknown: which encoding was not understood, for the error that names it
};

struct Entry {
  Cursor data;
  bool custom = false;
  int dialect = -1;
};

class Converter {
 public:
  Converter(const uint8_t* data, size_t size) {
    file_.base = data;
    file_.p = data;
    file_.end = data + size;
  }

  std::string run() {
    if (file_.left() < 4 || memcmp(file_.p, "ML\xEFR", 4) != 0) bad("missing magic number");
    file_.p += 4;
    version_ = file_.varint();
    if (version_ > 6) bad("bytecode version " + std::to_string(version_) + " is newer than this reader (6)");
    file_.cstring();   // producer
    std::map<int, Cursor> sections;
    while (!file_.empty()) {
      Cursor payload;
      int id = readSection(file_, payload);
      if (sections.count(id)) bad("duplicate section " + std::to_string(id));
      sections[id] = payload;
    }
    for (int need : {kString, kDialect, kAttrType, kAttrTypeOffset, kIR})
      if (!sections.count(need)) bad("missing section " + std::to_string(need));
    readStrings(sections[kString]);
    readDialects(sections[kDialect]);
    readOffsets(sections[kAttrTypeOffset], sections[kAttrType]);
    Cursor ir = sections[kIR];
    // the top-level block holds exactly the module op
    bool hasArgs;
    uint64_t numOps = ir.varintFlag(hasArgs);
    if (hasArgs || numOps != 1) bad("the top-level block must hold one builtin.module");
    scopes_.emplace_back();
    readOp(ir, 0, /*topLevel=*/true);
    out_ << "}\n";
    return out_.str();
  }

 private:
  Cursor file_;
  uint64_t version_ = 0;
  std::vector<std::string> strings_;
  std::vector<std::string> dialects_;
  struct OpName { int dialect; std::string name; };
  std::vector<OpName> opNames_;
  std::vector<Entry> attrEntries_, typeEntries_;
  std::vector<BAttr> attrs_;
  std::vector<BType> types_;
  std::ostringstream out_;
  int nextName_ = 0;

  struct Val { std::string name; int type = -1; };
  struct Scope { std::vector<Val> values; std::vector<size_t> next; };
  std::vector<Scope> scopes_;

  // ------------------------------------------------------------------ tables
  void readStrings(Cursor c) {
    uint64_t n = c.varint();
    std::vector<uint64_t> sizes(n);
    for (uint64_t k = 0; k < n; ++k) sizes[n - 1 - k] = c.varint();   // stored in reverse order
    strings_.resize(n);
    for (uint64_t k = 0; k < n; ++k) {
      if (sizes[k] == 0 || c.left() < sizes[k]) bad("string table is inconsistent");
      strings_[k] = std::string((const char*)c.p, (size_t)sizes[k] - 1);   // sizes count the terminating NUL
      c.p += sizes[k];
    }
  }
  const std::string& str(uint64_t idx) const {
    if (idx >= strings_.size()) bad("string index out of range");
    return strings_[idx];
  }

  void readDialects(Cursor c) {
    uint64_t n = c.varint();
    for (uint64_t k = 0; k < n; ++k) {
      if (version_ >= 1) {
        bool hasVersion;
        uint64_t nameIdx = c.varintFlag(hasVersion);
        dialects_.push_back(str(nameIdx));
        if (hasVersion) {
          Cursor payload;
          if (readSection(c, payload) != kDialectVersions) bad("expected a dialect version section");
        }
      } else {
        dialects_.push_back(str(c.varint()));
      }
    }
    if (version_ >= 4) c.varint();   // total number of op names
    while (!c.empty()) {
      uint64_t dialect = c.varint();
      uint64_t count = c.varint();
      if (dialect >= dialects_.size()) bad("dialect index out of range");
      for (uint64_t k = 0; k < count; ++k) {
        uint64_t nameIdx;
        if (version_ >= 5) { bool registered; nameIdx = c.varintFlag(registered); }
        else nameIdx = c.varint();
        opNames_.push_back({(int)dialect, str(nameIdx)});
      }
    }
  }

  void readOffsets(Cursor c, Cursor data) {
    uint64_t numAttrs = c.varint(), numTypes = c.varint();
    attrEntries_.resize(numAttrs);
    typeEntries_.resize(numTypes);
    size_t offset = 0;
    auto fill = [&](std::vector<Entry>& entries) {
      size_t at = 0;
      while (at < entries.size()) {
        uint64_t dialect = c.varint();
        uint64_t count = c.varint();
        if (dialect >= dialects_.size()) bad("dialect index out of range in the attribute table");
        for (uint64_t k = 0; k < count; ++k) {
          if (at >= entries.size()) bad("attribute table is inconsistent");
          Entry& e = entries[at++];
          uint64_t size = c.varintFlag(e.custom);
          if (offset + size > data.left()) bad("attribute data runs past its section");
          e.data.base = data.base;
          e.data.p = data.p + offset;
          e.data.end = e.data.p + size;
          e.dialect = (int)dialect;
          offset += (size_t)size;
        }
      }
    };
    fill(attrEntries_);
    fill(typeEntries_);
    attrs_.resize(numAttrs);
    types_.resize(numTypes);
  }

  // ------------------------------------------------------------------ types
  static const char* scalarName(int code) {
    switch (code) {
      case kBooleanT: return "i1";
      case kBF16T: return "bf16";
      case kF16T: return "f16";
      case kF32T: return "f32";
      case kF64T: return "f64";
      case kIndexT: return "index";
      case kSI4T: return "i4";
      case kSI8T: return "i8";
      case kSI16T: return "i16";
      case kSI32T: return "i32";
      case kSI64T: return "i64";
      case kUI4T: return "ui4";
      case kUI8T: return "ui8";
      case kUI16T: return "ui16";
      case kUI32T: return "ui32";
      case kUI64T: return "ui64";
      default: return nullptr;
    }
  }
  static int scalarBits(int code) {
    switch (code) {
      case kBooleanT: return 1;
      case kSI4T: case kUI4T: return 4;
      case kSI8T: case kUI8T: case kF8E4M3FNT: case kF8E5M2T: return 8;
      case kBF16T: case kF16T: case kSI16T: case kUI16T: return 16;
      case kF32T: case kSI32T: case kUI32T: return 32;
      case kF64T: case kSI64T: case kUI64T: case kIndexT: return 64;
      default: return 0;
    }
  }

  const BType& type(uint64_t idx) {
    if (idx >= types_.size()) bad("type index out of range");
    BType& t = types_[idx];
    if (t.decoded) return t;
    t.decoded = true;
    Entry& e = typeEntries_[idx];
    Cursor c = e.data;
    const std::string& dialect = dialects_[(size_t)e.dialect];
    if (!e.custom) {
      // stored as its textual form
      t.text = c.cstring();
      return t;
    }
    if (dialect != "vhlo") bad("type of dialect '" + dialect + "' in a binary encoding this reader does not know");
    t.vhlo = true;
    t.code = (int)c.varint();
    if (const char* s = scalarName(t.code)) { t.text = s; return t; }
    switch (t.code) {
      case kRankedTensorT:
      case kRankedTensorEncT: {
        if (t.code == kRankedTensorEncT) c.varint();   // encoding attribute: bounds of dynamic dims, not used for static shapes
        uint64_t rank = c.varint();
        for (uint64_t k = 0; k < rank; ++k) t.shape.push_back(c.svarint());
        t.elem = (int)c.varint();
        const std::string elemText = type((uint64_t)t.elem).text;   // (types_ never grows after the tables are read: `t` stays valid)
        std::string s = "tensor<";
        for (auto d : t.shape) {
          if (d < 0) bad("dynamic shapes are not supported");
          s += std::to_string(d) + "x";
        }
        t.text = s + elemText + ">";
        return t;
      }
      case kTokenT: t.text = "!stablehlo.token"; return t;
      case kFunctionT: {
        uint64_t ni = c.varint();
        for (uint64_t k = 0; k < ni; ++k) t.ins.push_back((int)c.varint());
        uint64_t no = c.varint();
        for (uint64_t k = 0; k < no; ++k) t.outs.push_back((int)c.varint());
        t.text = "function";
        return t;
      }
      case kTupleT: bad("tuple types are not supported");
      case kComplexT: bad("complex element types are not supported");
      case kUnrankedTensorT: bad("unranked tensors are not supported");
      case kF8E4M3FNT: case kF8E5M2T: bad("8-bit float element types are not supported");
      default: bad("vhlo type code " + std::to_string(t.code) + " is not supported");
    }
  }
  std::string typeText(uint64_t idx) {
    const BType& t = type(idx);
    if (t.text.empty() || t.text == "function") bad("a value has a type this reader cannot print");
    return t.text;
  }

  // ------------------------------------------------------------------ attributes
  const BAttr& attr(uint64_t idx) {
    if (idx >= attrs_.size()) bad("attribute index out of range");
    if (attrs_[idx].decoded) return attrs_[idx];
    BAttr a;
    a.decoded = true;
    Entry& e = attrEntries_[idx];
    Cursor c = e.data;
    const std::string& dialect = dialects_[(size_t)e.dialect];
    if (!e.custom) {
      a.kind = BAttr::Unknown;
      a.s = c.cstring();   // textual form (locations and the like): kept for diagnostics only
    } else if (dialect == "builtin") {
      uint64_t code = c.varint();
      switch (code) {
        case kBuiltinDictionaryAttr: {
          a.kind = BAttr::Dict;
          uint64_t n = c.varint();
          for (uint64_t k = 0; k < n; ++k) { int name = (int)c.varint(); int value = (int)c.varint(); a.pairs.push_back({name, value}); }
          break;
        }
        case kBuiltinStringAttr: a.kind = BAttr::String; a.s = str(c.varint()); break;
        case kBuiltinStringAttrWithType: a.kind = BAttr::String; a.s = str(c.varint()); break;
        case kBuiltinArrayAttr: {
          a.kind = BAttr::Array;
          uint64_t n = c.varint();
          for (uint64_t k = 0; k < n; ++k) a.elems.push_back((int)c.varint());
          break;
        }
        case kBuiltinFlatSymbolRefAttr: { a.kind = BAttr::Symbol; const BAttr& nm = attr(c.varint()); a.s = nm.s; break; }
        case kBuiltinUnitAttr: a.kind = BAttr::Unit; break;
        case kBuiltinTypeAttr: a.kind = BAttr::Type; a.type = (int)c.varint(); break;
        case kBuiltinIntegerAttr: {
          a.kind = BAttr::Int;
          a.type = (int)c.varint();
          a.i = c.svarint();   // widths up to 64 bits; one-byte form for widths <= 8 is not used by module attributes read here
          break;
        }
        default: a.kind = BAttr::Unknown; a.origin = "builtin attribute code " + std::to_string(code); break;   // locations and other attributes nothing here reads
      }
    } else if (dialect == "vhlo") {
      uint64_t code = c.varint();
      auto enumOf = [&](const char* kind, std::initializer_list<const char*> names) {
        a.kind = BAttr::Enum;
        a.enumKind = kind;
        uint64_t v = c.varint();
        if (v >= names.size()) bad(std::string("enum value out of range for ") + kind);
        a.s = *(names.begin() + v);
      };
      switch (code) {
        case kArrayV1: {
          a.kind = BAttr::Array;
          uint64_t n = c.varint();
          for (uint64_t k = 0; k < n; ++k) a.elems.push_back((int)c.varint());
          break;
        }
        case kBooleanV1: a.kind = BAttr::Bool; a.b = c.varint() != 0; break;
        case kComparisonDirectionV1: enumOf("comparison_direction", {"EQ", "NE", "GE", "GT", "LE", "LT"}); break;
        case kComparisonTypeV1: enumOf("comparison_type", {"NOTYPE", "FLOAT", "TOTALORDER", "SIGNED", "UNSIGNED"}); break;
        case kCustomCallApiVersionV1: enumOf("custom_call_api_version", {"API_VERSION_UNSPECIFIED", "API_VERSION_ORIGINAL", "API_VERSION_STATUS_RETURNING", "API_VERSION_STATUS_RETURNING_UNIFIED", "API_VERSION_TYPED_FFI"}); break;
        case kDictionaryV1: {
          a.kind = BAttr::Dict;
          uint64_t n = c.varint();
          for (uint64_t k = 0; k < n; ++k) { int name = (int)c.varint(); int value = (int)c.varint(); a.pairs.push_back({name, value}); }
          break;
        }
        case kFftTypeV1: enumOf("fft_type", {"FFT", "IFFT", "RFFT", "IRFFT"}); break;
        case kPrecisionV1: enumOf("precision", {"DEFAULT", "HIGH", "HIGHEST"}); break;
        case kRngAlgorithmV1: enumOf("rng_algorithm", {"DEFAULT", "THREE_FRY", "PHILOX"}); break;
        case kRngDistributionV1: enumOf("rng_distribution", {"INVALID", "UNIFORM", "NORMAL"}); break;
        case kTransposeV1: enumOf("transpose", {"TRANSPOSE_INVALID", "NO_TRANSPOSE", "TRANSPOSE", "ADJOINT"}); break;
        case kResultAccuracyModeV1: enumOf("result_accuracy_mode", {"DEFAULT", "HIGHEST", "TOLERANCE"}); break;
        case kFloatV1: {
          a.kind = BAttr::Float;
          a.type = (int)c.varint();
          int bits = scalarBits(type((uint64_t)a.type).code);
          a.bits = bits <= 8 ? c.byte() : (uint64_t)c.svarint();
          break;
        }
        case kIntegerV1: {
          a.kind = BAttr::Int;
          a.type = (int)c.varint();
          int bits = scalarBits(type((uint64_t)a.type).code);
          if (bits <= 0) bits = 64;
          a.i = bits <= 8 ? (int64_t)c.byte() : c.svarint();
          break;
        }
        case kStringV1: a.kind = BAttr::String; a.s = str(c.varint()); break;
        case kTensorV1: {
          a.kind = BAttr::Tensor;
          a.type = (int)c.varint();
          uint64_t n = c.varint();
          if (c.left() < n) bad("tensor attribute data runs past its entry");
          a.blob.assign(c.p, c.p + n);
          break;
        }
        case kTypeV1: a.kind = BAttr::Type; a.type = (int)c.varint(); break;
        case kTypeExtensionsV1: {
          a.kind = BAttr::Ints;
          uint64_t n = c.varint();
          for (uint64_t k = 0; k < n; ++k) a.ints.push_back(c.svarint());
          break;
        }
        default: a.kind = BAttr::Unknown; a.origin = "vhlo attribute code " + std::to_string(code); break;   // output_operand_alias, result_accuracy: nothing on this path reads them
      }
    } else {
      a.kind = BAttr::Unknown;
      a.origin = "an attribute of dialect '" + dialect + "'";
    }
    attrs_[idx] = std::move(a);
    return attrs_[idx];
  }

  // integer elements of a tensor attribute (splat expanded)
  std::vector<int64_t> tensorInts(const BAttr& a) {
    if (a.kind != BAttr::Tensor) bad("expected a tensor attribute of integers");
    const BType& t = type((uint64_t)a.type);
    int64_t n = 1;
    for (auto d : t.shape) n *= d;
    int code = type((uint64_t)t.elem).code;
    int bits = scalarBits(code);
    std::vector<int64_t> out;
    if (bits == 1) {
      bool packed = (int64_t)a.blob.size() != n && (int64_t)a.blob.size() == (n + 7) / 8;
      for (int64_t k = 0; k < n; ++k) {
        if (a.blob.size() == 1 && n != 1 && !packed) out.push_back(a.blob[0] ? 1 : 0);
        else if (packed) out.push_back((a.blob[(size_t)k / 8] >> (k % 8)) & 1);
        else out.push_back(a.blob[(size_t)k] ? 1 : 0);
      }
      if (n == 1 && !a.blob.empty()) out.assign(1, a.blob[0] ? 1 : 0);
      return out;
    }
    size_t esz = (size_t)bits / 8;
    if (esz == 0 || (code != kSI8T && code != kSI16T && code != kSI32T && code != kSI64T && code != kUI8T && code != kUI16T && code != kUI32T &&
                     code != kUI64T && code != kIndexT))
      bad("expected integer elements");
    bool splat = a.blob.size() == esz && n != 1;
    if (!splat && a.blob.size() != (size_t)n * esz) bad("tensor attribute has the wrong size");
    bool isSigned = code == kSI8T || code == kSI16T || code == kSI32T || code == kSI64T || code == kIndexT;
    for (int64_t k = 0; k < n; ++k) {
      const uint8_t* q = a.blob.data() + (splat ? 0 : (size_t)k * esz);
      uint64_t u = 0;
      memcpy(&u, q, esz);
      int64_t v = (int64_t)u;
      if (isSigned && esz < 8 && ((u >> (8 * esz - 1)) & 1)) v = (int64_t)(u | ~((1ull << (8 * esz)) - 1));
      out.push_back(v);
    }
    return out;
  }

  static std::string list(const std::vector<int64_t>& v, const char* open = "[", const char* close = "]") {
    std::string s = open;
    for (size_t k = 0; k < v.size(); ++k) s += (k ? ", " : "") + std::to_string(v[k]);
    return s + close;
  }
  static std::string i64Array(const std::vector<int64_t>& v) {
    if (v.empty()) return "array<i64>";
    return "array<i64: " + list(v, "", "") + ">";
  }
  static std::string quoted(const std::string& s) {
    std::string o = "\"";
    static const char* hex = "0123456789ABCDEF";
    for (unsigned char ch : s) {
      if (ch == '"' || ch == '\\' || ch < 0x20 || ch >= 0x7F) { o += '\\'; o += hex[ch >> 4]; o += hex[ch & 15]; }
      else o += (char)ch;
    }
    return o + "\"";
  }

  // generic text of an attribute value
  std::string attrText(const BAttr& a) {
    switch (a.kind) {
      case BAttr::Bool: return a.b ? "true" : "false";
      case BAttr::Unit: return "unit";
      case BAttr::Int: {
        std::string t = a.type >= 0 ? type((uint64_t)a.type).text : std::string("i64");
        if (t.empty()) t = "i64";
        return std::to_string(a.i) + " : " + t;
      }
      case BAttr::Float: {
        const BType& t = type((uint64_t)a.type);
        char buf[64];
        if (t.code == kF32T) { uint32_t u = (uint32_t)a.bits; float f; memcpy(&f, &u, 4); snprintf(buf, sizeof buf, "%.9g", (double)f); }
        else if (t.code == kF64T) { double d; memcpy(&d, &a.bits, 8); snprintf(buf, sizeof buf, "%.17g", d); }
        else { snprintf(buf, sizeof buf, "0x%llX", (unsigned long long)a.bits); }
        std::string s = buf;
        if (s.find_first_of(".eEnx") == std::string::npos) s += ".0";
        return s + " : " + t.text;
      }
      case BAttr::String: return quoted(a.s);
      case BAttr::Symbol: return "@" + quoted(a.s);
      case BAttr::Enum: return "#stablehlo<" + a.enumKind + " " + a.s + ">";
      case BAttr::Type: return typeText((uint64_t)a.type);
      case BAttr::Ints: return list(a.ints);
      case BAttr::Array: {
        std::string s = "[";
        for (size_t k = 0; k < a.elems.size(); ++k) s += (k ? ", " : "") + attrText(attr((uint64_t)a.elems[k]));
        return s + "]";
      }
      case BAttr::Dict: {
        std::string s = "{";
        for (size_t k = 0; k < a.pairs.size(); ++k) {
          s += (k ? ", " : "") + quoted(attr((uint64_t)a.pairs[k].first).s) + " = " + attrText(attr((uint64_t)a.pairs[k].second));
        }
        return s + "}";
      }
      case BAttr::Tensor: return denseText(a);
      default: return "unit";
    }
  }

  std::string denseText(const BAttr& a) {
    const BType& t = type((uint64_t)a.type);
    const BType& el = type((uint64_t)t.elem);
    int64_t n = 1;
    for (auto d : t.shape) n *= d;
    if (el.code == kBooleanT) {
      // one value per element as text: the in-memory forms (bit-packed, one byte per element, 0xFF splats) all occur
      std::vector<int64_t> v = tensorInts(a);
      bool same = true;
      for (auto x : v) same = same && x == v[0];
      if (same && !v.empty()) return std::string("dense<") + (v[0] ? "true" : "false") + "> : " + t.text;
      std::string s = "dense<\"0x";
      static const char* hex = "0123456789ABCDEF";
      for (auto x : v) { s += hex[0]; s += hex[x ? 1 : 0]; }
      return s + "\"> : " + t.text;
    }
    std::string s = "dense<\"0x";
    static const char* hex = "0123456789ABCDEF";
    s.reserve(a.blob.size() * 2 + 32);
    for (uint8_t b : a.blob) { s += hex[b >> 4]; s += hex[b & 15]; }
    (void)n;
    return s + "\"> : " + t.text;
  }

  // ------------------------------------------------------------------ IR
  std::string fresh() { return "%v" + std::to_string(nextName_++); }

  Val& valueAt(uint64_t idx) {
    Scope& sc = scopes_.back();
    if (idx >= sc.values.size()) bad("operand refers to a value outside its scope");
    return sc.values[idx];
  }
  void defineValue(const std::string& name, int typeIdx) {
    Scope& sc = scopes_.back();
    if (sc.next.empty() || sc.next.back() >= sc.values.size()) bad("a region defines more values than it declares");
    sc.values[sc.next.back()++] = Val{name, typeIdx};
  }
  void pushRegionValues(uint64_t numValues) {
    Scope& sc = scopes_.back();
    sc.next.push_back(sc.values.size());
    sc.values.resize(sc.values.size() + (size_t)numValues);
  }
  void popRegionValues(uint64_t numValues) {
    Scope& sc = scopes_.back();
    sc.values.resize(sc.values.size() - (size_t)numValues);
    sc.next.pop_back();
  }

  static std::string baseName(const std::string& versioned) {
    size_t u = versioned.rfind("_v");
    if (u == std::string::npos || u + 2 >= versioned.size()) return versioned;
    for (size_t k = u + 2; k < versioned.size(); ++k) if (!isdigit((unsigned char)versioned[k])) return versioned;
    return versioned.substr(0, u);
  }

  const BAttr* find(const BAttr* dict, const char* key) {
    if (!dict) return nullptr;
    for (auto& kv : dict->pairs) if (attr((uint64_t)kv.first).s == key) return &attr((uint64_t)kv.second);
    return nullptr;
  }
  std::vector<int64_t> intsOf(const BAttr* a) {
    if (!a) return {};
    if (a->kind == BAttr::Tensor) return tensorInts(*a);
    if (a->kind == BAttr::Ints) return a->ints;
    if (a->kind == BAttr::Int) return {a->i};
    if (a->kind == BAttr::Array) {
      std::vector<int64_t> out;
      for (int e : a->elems) { const BAttr& x = attr((uint64_t)e); out.push_back(x.kind == BAttr::Bool ? (x.b ? 1 : 0) : x.i); }
      return out;
    }
    return {};
  }

  // attribute dictionary of a vhlo op as the generic StableHLO text form parser.cc normalises
  std::string opAttrs(const std::string& name, const BAttr* dict) {
    if (!dict) return "";
    std::vector<std::string> parts;
    std::vector<std::string> done;
    // an attribute the op's meaning depends on must have been understood: one whose encoding this reader does not know
    // is a compile error that names it, never a silent default
    auto known = [&](const std::string& k, const BAttr* a) {
      if (a && a->kind == BAttr::Unknown)
        bad("attribute '" + k + "' of vhlo." + name + " is encoded as " + (a->origin.empty() ? std::string("a textual attribute") : a->origin) +
            ", which this reader does not know");
      return a;
    };
    auto take = [&](const char* k) { done.push_back(k); return known(k, find(dict, k)); };
    auto dims = [&](const char* k) { return list(intsOf(take(k))); };
    if (name == "dot_general") {
      parts.push_back("dot_dimension_numbers = #stablehlo.dot<lhs_batching_dimensions = " + dims("lhs_batching_dimensions") + ", rhs_batching_dimensions = " +
                      dims("rhs_batching_dimensions") + ", lhs_contracting_dimensions = " + dims("lhs_contracting_dimensions") +
                      ", rhs_contracting_dimensions = " + dims("rhs_contracting_dimensions") + ">");
    } else if (name == "gather") {
      std::string d = "dimension_numbers = #stablehlo.gather<offset_dims = " + dims("offset_dims") + ", collapsed_slice_dims = " + dims("collapsed_slice_dims");
      if (find(dict, "operand_batching_dims")) d += ", operand_batching_dims = " + dims("operand_batching_dims") + ", start_indices_batching_dims = " + dims("start_indices_batching_dims");
      d += ", start_index_map = " + dims("start_index_map") + ", index_vector_dim = " + std::to_string(intsOf(take("index_vector_dim")).at(0)) + ">";
      parts.push_back(d);
      parts.push_back("slice_sizes = " + i64Array(intsOf(take("slice_sizes"))));
    } else if (name == "scatter") {
      std::string d = "scatter_dimension_numbers = #stablehlo.scatter<update_window_dims = " + dims("update_window_dims") + ", inserted_window_dims = " + dims("inserted_window_dims");
      if (find(dict, "input_batching_dims")) d += ", input_batching_dims = " + dims("input_batching_dims") + ", scatter_indices_batching_dims = " + dims("scatter_indices_batching_dims");
      d += ", scatter_dims_to_operand_dims = " + dims("scatter_dims_to_operand_dims") + ", index_vector_dim = " + std::to_string(intsOf(take("index_vector_dim")).at(0)) + ">";
      parts.push_back(d);
    } else if (name == "convolution") {
      auto spatial = [&](const char* k) { return intsOf(take(k)); };
      auto lhsSp = spatial("input_spatial_dimensions"), rhsSp = spatial("kernel_spatial_dimensions"), outSp = spatial("output_spatial_dimensions");
      size_t rank = lhsSp.size() + 2;
      auto spec = [&](int64_t a, const char* an, int64_t b, const char* bn, const std::vector<int64_t>& sp) {
        std::vector<std::string> names(rank, "?");
        if (a < 0 || b < 0 || (size_t)a >= rank || (size_t)b >= rank) bad("convolution dimension numbers are out of range");
        names[(size_t)a] = an;
        names[(size_t)b] = bn;
        for (size_t k = 0; k < sp.size(); ++k) { if (sp[k] < 0 || (size_t)sp[k] >= rank) bad("convolution dimension numbers are out of range"); names[(size_t)sp[k]] = std::to_string(k); }
        std::string s = "[";
        for (size_t k = 0; k < rank; ++k) s += (k ? ", " : "") + names[k];
        return s + "]";
      };
      std::string d = "dimension_numbers = #stablehlo.conv<" +
                      spec(intsOf(take("input_batch_dimension")).at(0), "b", intsOf(take("input_feature_dimension")).at(0), "f", lhsSp) + "x" +
                      spec(intsOf(take("kernel_input_feature_dimension")).at(0), "i", intsOf(take("kernel_output_feature_dimension")).at(0), "o", rhsSp) + "->" +
                      spec(intsOf(take("output_batch_dimension")).at(0), "b", intsOf(take("output_feature_dimension")).at(0), "f", outSp) + ">";
      parts.push_back(d);
      if (auto* a = take("window_strides")) if (!intsOf(a).empty()) parts.push_back("window_strides = " + i64Array(intsOf(a)));
      if (auto* a = take("lhs_dilation")) if (!intsOf(a).empty()) parts.push_back("lhs_dilation = " + i64Array(intsOf(a)));
      if (auto* a = take("rhs_dilation")) if (!intsOf(a).empty()) parts.push_back("rhs_dilation = " + i64Array(intsOf(a)));
      if (auto* a = take("padding")) if (!intsOf(a).empty()) parts.push_back("padding = " + i64Array(intsOf(a)));   // flattened lo/hi pairs
      if (auto* a = take("window_reversal")) {
        auto v = intsOf(a);
        if (!v.empty()) {
          std::string s = "window_reversal = array<i1: ";
          for (size_t k = 0; k < v.size(); ++k) s += std::string(k ? ", " : "") + (v[k] ? "true" : "false");
          parts.push_back(s + ">");
        }
      }
    } else if (name == "func" || name == "call" || name == "composite") {
      return "";   // handled by the callers
    }
    // everything else keeps its name; one-dimensional integer tensors print as arrays, which is what the text forms hold
    static const char* skip[] = {"precision_config", "lhs_precision_type", "rhs_precision_type", "accumulation_type", "lhs_component_count",
                                 "rhs_component_count", "num_primitive_operations", "allow_imprecise_accumulation", "result_accuracy",
                                 "operand_layouts", "result_layouts", "output_operand_aliases", "called_computations", "api_version"};
    for (auto& kv : dict->pairs) {
      const std::string& k = attr((uint64_t)kv.first).s;
      bool handled = false;
      for (auto& d : done) if (d == k) handled = true;
      for (auto* s : skip) if (k == s) handled = true;
      if (handled) continue;
      const BAttr& v = attr((uint64_t)kv.second);
      known(k, &v);
      if (name == "compare" && k == "compare_type" && v.s == "NOTYPE") continue;
      if (name == "custom_call" && k == "backend_config" && v.kind != BAttr::String) continue;
      std::string text;
      if (v.kind == BAttr::Tensor && name != "constant") {
        const BType& t = type((uint64_t)v.type);
        const BType& el = type((uint64_t)t.elem);
        if (k != "replica_groups" && t.shape.size() <= 2 && el.code != kBooleanT && el.code != kF32T && el.code != kF64T && el.code != kBF16T && el.code != kF16T) text = i64Array(tensorInts(v));
        else text = denseText(v);
      } else {
        text = attrText(v);
      }
      parts.push_back(k + " = " + text);
    }
    if (parts.empty()) return "";
    std::string s = " <{";
    for (size_t k = 0; k < parts.size(); ++k) s += (k ? ", " : "") + parts[k];
    return s + "}>";
  }

  void indent(int depth) { for (int k = 0; k < depth; ++k) out_ << "  "; }

  // one region: `{ ^bb0(args): ops }`; `header` (optional) receives the block arguments instead of printing them
  void readRegion(Cursor& c, int depth, std::vector<Val>* header) {
    uint64_t numBlocks = c.varint();
    if (numBlocks == 0) { if (!header) out_ << "{\n"; return; }
    if (numBlocks != 1) bad("regions with several blocks are not supported");
    uint64_t numValues = c.varint();
    pushRegionValues(numValues);
    bool hasArgs;
    uint64_t numOps = c.varintFlag(hasArgs);
    std::vector<Val> args;
    if (hasArgs) {
      uint64_t n = c.varint();
      for (uint64_t k = 0; k < n; ++k) {
        uint64_t typeIdx;
        if (version_ >= 4) {
          bool hasLoc;
          typeIdx = c.varintFlag(hasLoc);
          if (hasLoc) c.varint();
        } else {
          typeIdx = c.varint();
          c.varint();
        }
        Val v{fresh(), (int)typeIdx};
        defineValue(v.name, v.type);
        args.push_back(v);
      }
      if (version_ >= 3 && c.byte() != 0) bad("use-list orders are not supported");
    }
    if (header) {
      *header = args;
    } else {
      out_ << "{\n";
      if (!args.empty()) {
        indent(depth);
        out_ << "^bb0(";
        for (size_t k = 0; k < args.size(); ++k) out_ << (k ? ", " : "") << args[k].name << ": " << typeText((uint64_t)args[k].type);
        out_ << "):\n";
      }
    }
    for (uint64_t k = 0; k < numOps; ++k) readOp(c, depth, false);
    popRegionValues(numValues);
  }

  void readOp(Cursor& c, int depth, bool topLevel) {
    uint64_t nameIdx = c.varint();
    if (nameIdx >= opNames_.size()) bad("operation name index out of range");
    const OpName& on = opNames_[nameIdx];
    const std::string& dialect = dialects_[(size_t)on.dialect];
    uint8_t mask = c.byte();
    c.varint();   // location
    const BAttr* dict = nullptr;
    if (mask & 0x01) {
      const BAttr& d = attr(c.varint());
      if (d.kind != BAttr::Dict) bad("an operation's attributes are not a dictionary");
      dict = &d;
    }
    if (mask & 0x40) {
      // Native properties (container version 5 and later).  VHLO keeps every attribute in the dictionary, so in a
      // portable artifact only builtin.module has any (its symbol name and visibility, which nothing here needs):
      // the index into the properties section is read and dropped.
      if (!(dialect == "builtin" && on.name == "module"))
        bad("operations with native properties are not supported (" + dialect + "." + on.name + ")");
      c.varint();
    }
    std::vector<int> resultTypes;
    if (mask & 0x02) {
      uint64_t n = c.varint();
      for (uint64_t k = 0; k < n; ++k) resultTypes.push_back((int)c.varint());
    }
    std::vector<Val> operands;
    if (mask & 0x04) {
      uint64_t n = c.varint();
      for (uint64_t k = 0; k < n; ++k) {
        Val& v = valueAt(c.varint());
        if (v.name.empty()) bad("use of a value before its definition");
        operands.push_back(v);
      }
    }
    if (mask & 0x08) bad("operations with successors are not supported");
    if (mask & 0x20) bad("use-list orders are not supported");
    uint64_t numRegions = 0;
    bool isolated = false;
    if (mask & 0x10) numRegions = c.varintFlag(isolated);

    // results are defined before the regions are read (regions never use them, but the numbering follows definition order)
    std::vector<Val> results;
    for (int t : resultTypes) {
      Val v{fresh(), t};
      results.push_back(v);
    }

    auto regionCursor = [&](Cursor& outer) -> Cursor {
      // regions of an op that is isolated from above are sections of their own since version 2
      if (isolated && version_ >= 2) {
        Cursor payload;
        if (readSection(outer, payload) != kIR) bad("expected an IR section for an isolated region");
        return payload;
      }
      return Cursor();
    };

    if (dialect == "builtin" && on.name == "module") {
      if (!topLevel) bad("nested modules are not supported");
      if (numRegions != 1) bad("builtin.module must have one region");
      // the device counts are the only module attributes the compiler reads (partition_id and replica_id need them)
      out_ << "module";
      const char* sep = " attributes {";
      for (const char* key : {"mhlo.num_partitions", "mhlo.num_replicas"})
        if (const BAttr* v = find(dict, key); v && v->kind == BAttr::Int) {
          out_ << sep << key << " = " << v->i << " : i32";
          sep = ", ";
        }
      out_ << (sep[0] == ',' ? "} {\n" : " {\n");
      Cursor rc = regionCursor(c);
      Cursor& use = (isolated && version_ >= 2) ? rc : c;
      if (isolated) scopes_.emplace_back();
      uint64_t numBlocks = use.varint();
      if (numBlocks == 1) {
        uint64_t numValues = use.varint();
        pushRegionValues(numValues);
        bool hasArgs;
        uint64_t numOps = use.varintFlag(hasArgs);
        if (hasArgs) bad("the module block has arguments");
        for (uint64_t k = 0; k < numOps; ++k) readOp(use, 1, false);
        popRegionValues(numValues);
      } else if (numBlocks != 0) {
        bad("the module region must have one block");
      }
      if (isolated) scopes_.pop_back();
      return;
    }
    if (dialect != "vhlo") bad("operation of dialect '" + dialect + "' (" + on.name + "): a portable artifact holds vhlo operations only");
    const std::string name = baseName(on.name);
    for (auto& v : results) defineValue(v.name, v.type);

    if (name == "func") {
      const BAttr* symName = find(dict, "sym_name");
      const BAttr* fnType = find(dict, "function_type");
      const BAttr* vis = find(dict, "sym_visibility");
      const BAttr* argAttrs = find(dict, "arg_attrs");
      if (!symName || !fnType || fnType->kind != BAttr::Type) bad("vhlo.func without a name or a type");
      const BType ft = type((uint64_t)fnType->type);
      if (numRegions != 1) bad("vhlo.func must have one region");
      Cursor rc = regionCursor(c);
      Cursor& use = (isolated && version_ >= 2) ? rc : c;
      if (isolated) scopes_.emplace_back();
      std::vector<Val> args;
      std::ostringstream saved;
      saved.swap(out_);                    // the body is printed first (its argument names are needed for the header)
      readRegion(use, depth + 1, &args);
      std::string body = out_.str();
      out_.swap(saved);
      if (isolated) scopes_.pop_back();
      indent(depth);
      out_ << "func.func " << ((vis && vis->s == "private") ? "private" : "public") << " @" << quoted(symName->s) << "(";
      for (size_t k = 0; k < args.size(); ++k) {
        out_ << (k ? ", " : "") << args[k].name << ": " << typeText((uint64_t)args[k].type);
        if (argAttrs && argAttrs->kind == BAttr::Array && k < argAttrs->elems.size()) {
          const BAttr& ad = attr((uint64_t)argAttrs->elems[k]);
          std::string parts;
          if (ad.kind == BAttr::Dict)
            for (auto& kv : ad.pairs) {
              const std::string& key = attr((uint64_t)kv.first).s;
              const BAttr& val = attr((uint64_t)kv.second);
              if (key == "tf.aliasing_output" && val.kind == BAttr::Int) parts += (parts.empty() ? "" : ", ") + key + " = " + std::to_string(val.i) + " : i32";
              if (key == "jax.buffer_donor" && val.kind == BAttr::Bool && val.b) parts += (parts.empty() ? "" : ", ") + key + " = true";
            }
          if (!parts.empty()) out_ << " {" << parts << "}";
        }
      }
      out_ << ") -> (";
      for (size_t k = 0; k < ft.outs.size(); ++k) out_ << (k ? ", " : "") << typeText((uint64_t)ft.outs[k]);
      out_ << ") {\n" << body;
      indent(depth);
      out_ << "}\n";
      return;
    }

    indent(depth);
    if (!results.empty()) {
      for (size_t k = 0; k < results.size(); ++k) out_ << (k ? ", " : "") << results[k].name;
      out_ << " = ";
    }
    std::string full;
    std::string attrsText;
    if (name == "return") full = "stablehlo.return";
    else if (name == "call") {
      full = "func.call";
      const BAttr* callee = find(dict, "callee");
      if (!callee) bad("vhlo.call without a callee");
      attrsText = " <{callee = @" + quoted(callee->s) + "}>";
    } else if (name == "composite") {
      full = "stablehlo.composite";
      const BAttr* nm = find(dict, "name");
      const BAttr* dec = find(dict, "decomposition");
      if (!dec) bad("vhlo.composite without a decomposition");
      attrsText = " <{decomposition = @" + quoted(dec->s) + ", name = " + quoted(nm ? nm->s : std::string()) + "}>";
    } else {
      full = "stablehlo." + name;
      attrsText = opAttrs(name, dict);
    }
    out_ << "\"" << full << "\"(";
    for (size_t k = 0; k < operands.size(); ++k) out_ << (k ? ", " : "") << operands[k].name;
    out_ << ")" << attrsText;
    if (numRegions > 0) {
      out_ << " (";
      for (uint64_t r = 0; r < numRegions; ++r) {
        if (r) out_ << ", ";
        Cursor rc = regionCursor(c);
        Cursor& use = (isolated && version_ >= 2) ? rc : c;
        if (isolated) scopes_.emplace_back();
        readRegion(use, depth + 2, nullptr);
        if (isolated) scopes_.pop_back();
        indent(depth + 1);
        out_ << "}";
      }
      out_ << ")";
    }
    out_ << " : (";
    for (size_t k = 0; k < operands.size(); ++k) out_ << (k ? ", " : "") << typeText((uint64_t)operands[k].type);
    out_ << ") -> (";
    for (size_t k = 0; k < results.size(); ++k) out_ << (k ? ", " : "") << typeText((uint64_t)results[k].type);
    out_ << ")\n";
  }
};

}  // namespace

bool isMlirBytecode(const char* data, size_t size) {
  return size >= 4 && data[0] == 'M' && data[1] == 'L' && (unsigned char)data[2] == 0xEF && data[3] == 'R';
}

std::string vhloBytecodeToStableHLOText(const char* data, size_t size) {
  Converter c((const uint8_t*)data, size);
  return c.run();
}

}  // namespace mi355
