// ByRE text reader.  The reference parses ByRE with MLIR (runtime/lib/core/ir/ir.cc:128-166);
// MLIR is not available to this runtime, so the textual forms the ByteIR compiler prints for the
// ops on the hot path are read directly:
//
//   module attributes {byre.container_module} {
//     func.func @name(%arg0 : memref<1x128x3x32xf16, "cuda"> {byre.argname = "Q", byre.argtype = 2: i32}, ...)
//         attributes {byre.entry_point} {
//       %0 = memref.alloc() : memref<32xf32, "cuda">
//       %1 = "byre.alias"(%0) {device = "cuda", offset = 16 : i64} : (memref<...>) -> memref<...>
//       byre.compute @ReduceSumOp_f32_f32(%arg0, %1) {dimensions = dense<[0, 1]> : tensor<2xi64>, ...} : memref<...>, memref<...>
//       "byre.custom"(%arg0, ...) {callee = "custom", lib_path = "...", extra_args = [1 : i64, 0.5 : f32]} : (...) -> ()
//       return
//     }
//   }
//
// Examples in the reference: runtime/test/test_files/flash_attn_fwd.mlir,
// resnet18_fw_bw_host_cuda.mlir:59,178,185,300, group_allocation_hook_cpu_group.mlir:4.
#include <cctype>
#include <cstdlib>
#include <fstream>
#include <functional>
#include <sstream>

#include "brt.h"

namespace brt {
namespace ir {
namespace {

struct ParseError : std::runtime_error {
  using std::runtime_error::runtime_error;
};

class Lexer {
public:
  explicit Lexer(const std::string &t) : t_(t) {}
  int line() const { return line_; }

  void SkipWs() {
    for (;;) {
      while (pos_ < t_.size() && std::isspace((unsigned char)t_[pos_])) {
        if (t_[pos_] == '\n') ++line_;
        ++pos_;
      }
      if (pos_ + 1 < t_.size() && t_[pos_] == '/' && t_[pos_ + 1] == '/') {
        while (pos_ < t_.size() && t_[pos_] != '\n') ++pos_;
        continue;
      }
      break;
    }
  }
  bool Eof() { SkipWs(); return pos_ >= t_.size(); }
  char Peek() { SkipWs(); return pos_ < t_.size() ? t_[pos_] : '\0'; }
  bool PeekIs(const std::string &s) { SkipWs(); return t_.compare(pos_, s.size(), s) == 0; }
  bool Accept(const std::string &s) {
    if (!PeekIs(s)) return false;
    pos_ += s.size();
    return true;
  }
  void Expect(const std::string &s) {
    if (!Accept(s)) Fail("expected '" + s + "'");
  }
  [[noreturn]] void Fail(const std::string &what) {
    SkipWs();
    std::string near = t_.substr(pos_, 40);
    for (auto &c : near) if (c == '\n') c = ' ';
    throw ParseError("line " + std::to_string(line_) + ": " + what + " near '" + near + "'");
  }
  // identifier characters of MLIR bare ids, including dots and dollars
  std::string Ident() {
    SkipWs();
    size_t b = pos_;
    while (pos_ < t_.size() && (std::isalnum((unsigned char)t_[pos_]) || t_[pos_] == '_' || t_[pos_] == '.' || t_[pos_] == '$'))
      ++pos_;
    if (b == pos_) Fail("expected identifier");
    return t_.substr(b, pos_ - b);
  }
  std::string ValueName() {  // %name
    SkipWs();
    if (Peek() != '%') Fail("expected SSA value");
    ++pos_;
    return "%" + Ident();
  }
  std::string String() {
    SkipWs();
    if (Peek() != '"') Fail("expected string");
    ++pos_;
    std::string out;
    while (pos_ < t_.size() && t_[pos_] != '"') {
      if (t_[pos_] == '\\' && pos_ + 1 < t_.size()) ++pos_;
      out.push_back(t_[pos_++]);
    }
    if (pos_ >= t_.size()) Fail("unterminated string");
    ++pos_;
    return out;
  }
  // number token; *is_float set when it has '.', 'e' or is inf/nan
  std::string Number(bool *is_float) {
    SkipWs();
    size_t b = pos_;
    if (pos_ < t_.size() && (t_[pos_] == '-' || t_[pos_] == '+')) ++pos_;
    *is_float = false;
    if (t_.compare(pos_, 2, "0x") == 0) {  // hex literal (also used for float bit patterns)
      pos_ += 2;
      while (pos_ < t_.size() && std::isxdigit((unsigned char)t_[pos_])) ++pos_;
      return t_.substr(b, pos_ - b);
    }
    while (pos_ < t_.size()) {
      const char c = t_[pos_];
      if (std::isdigit((unsigned char)c)) { ++pos_; continue; }
      if (c == '.') { *is_float = true; ++pos_; continue; }
      if ((c == 'e' || c == 'E') && pos_ > b && (std::isdigit((unsigned char)t_[pos_ - 1]) || t_[pos_ - 1] == '.') &&
          pos_ + 1 < t_.size() &&
          (std::isdigit((unsigned char)t_[pos_ + 1]) ||
           ((t_[pos_ + 1] == '-' || t_[pos_ + 1] == '+') && pos_ + 2 < t_.size() && std::isdigit((unsigned char)t_[pos_ + 2])))) {
        *is_float = true;
        pos_ += 2;  // the exponent marker and its sign or first digit
        continue;
      }
      break;
    }
    if (b == pos_ || (pos_ == b + 1 && !std::isdigit((unsigned char)t_[b]))) Fail("expected number");
    return t_.substr(b, pos_ - b);
  }
  // plain decimal digits (memref / tensor dimensions, where "0x16" is two dimensions, not hex)
  int64_t Digits() {
    SkipWs();
    size_t b = pos_;
    while (pos_ < t_.size() && std::isdigit((unsigned char)t_[pos_])) ++pos_;
    if (b == pos_) Fail("expected dimension");
    return std::strtoll(t_.substr(b, pos_ - b).c_str(), nullptr, 10);
  }
  // skips a balanced <...> group (used for types we do not interpret, e.g. tensor<2xi64>)
  void SkipAngle() {
    Expect("<");
    int depth = 1;
    while (pos_ < t_.size() && depth) {
      if (t_[pos_] == '<') ++depth;
      else if (t_[pos_] == '>') --depth;
      else if (t_[pos_] == '\n') ++line_;
      ++pos_;
    }
    if (depth) Fail("unbalanced '<'");
  }

private:
  const std::string &t_;
  size_t pos_ = 0;
  int line_ = 1;
};

DTypeEnum ParseElemType(const std::string &s) {
  if (s == "f32") return DTypeEnum::Float32;
  if (s == "f16") return DTypeEnum::Float16;
  if (s == "bf16") return DTypeEnum::BFloat16;
  if (s == "f64") return DTypeEnum::Float64;
  if (s == "i64" || s == "ui64" || s == "si64" || s == "index") return DTypeEnum::Int64;
  if (s == "i32" || s == "ui32" || s == "si32") return DTypeEnum::Int32;
  if (s == "i16" || s == "ui16") return DTypeEnum::Int16;
  if (s == "i8" || s == "si8") return DTypeEnum::Int8;
  if (s == "ui8") return DTypeEnum::UInt8;
  if (s == "i1") return DTypeEnum::Bool;
  return DTypeEnum::Invalid;
}

class Parser {
public:
  Parser(const std::string &text, ByREHandle *h) : lx_(text), h_(h) {}

  void Run() {
    if (lx_.Accept("module")) {
      if (lx_.Accept("@")) {  // module @IrToMhlo.2452 attributes {...}: the symbol name is not used
        if (lx_.Peek() == '"') lx_.String(); else lx_.Ident();
      }
      if (lx_.Accept("attributes")) ParseAttrDict();
      lx_.Expect("{");
      ParseFunc();
      lx_.Expect("}");
    } else {
      ParseFunc();
    }
  }

private:
  // memref<4x?x8xf32, "cuda">; dynamic sizes are rejected (static shapes only on this path)
  MemRefType ParseMemRef() {
    lx_.Expect("memref");
    lx_.Expect("<");
    MemRefType t;
    for (;;) {
      const char c = lx_.Peek();
      if (std::isdigit((unsigned char)c)) {
        // a dimension: digits followed by 'x' ("1x128x3x32xf16")
        t.shape.push_back(lx_.Digits());
        lx_.Expect("x");
      } else if (c == '?') {
        lx_.Fail("dynamic memref shapes are not supported");
      } else {
        break;
      }
    }
    const std::string et = lx_.Ident();
    t.dtype = ParseElemType(et);
    if (t.dtype == DTypeEnum::Invalid) lx_.Fail("unsupported element type '" + et + "'");
    if (lx_.Accept(",")) {
      if (lx_.Peek() == '"') t.space = lx_.String();
      else lx_.Fail("only string memory spaces are supported");
    }
    lx_.Expect(">");
    return t;
  }

  void SkipType() {  // a type we do not need: memref<...>, tensor<...>, iN, fN, index, ()
    if (lx_.Accept("(")) { lx_.Expect(")"); return; }
    lx_.Ident();
    if (lx_.Peek() == '<') lx_.SkipAngle();
  }

  Scalar ParseNumberWithType() {
    Scalar s;
    bool is_float;
    const std::string n = lx_.Number(&is_float);
    std::string ty;
    if (lx_.Accept(":")) ty = lx_.Ident();
    if (is_float || (!ty.empty() && (ty[0] == 'f' || ty == "bf16"))) {
      s.is_float = true;
      s.f = std::strtod(n.c_str(), nullptr);
      s.i = (int64_t)s.f;
    } else {
      s.i = std::strtoll(n.c_str(), nullptr, 0);
      s.f = (double)s.i;
    }
    return s;
  }

  Attr ParseAttrValue() {
    Attr a;
    const char c = lx_.Peek();
    if (c == '"') {
      a.kind = Attr::String;
      a.s = lx_.String();
      if (lx_.Accept(":")) SkipType();
    } else if (c == '@') {
      lx_.Expect("@");
      a.kind = Attr::String;
      a.s = lx_.Peek() == '"' ? lx_.String() : lx_.Ident();
    } else if (c == '[') {
      lx_.Expect("[");
      a.kind = Attr::Array;
      if (!lx_.Accept("]")) {
        do {
          const char e = lx_.Peek();
          if (e == '-' || e == '+' || std::isdigit((unsigned char)e)) {
            a.elems.push_back(ParseNumberWithType());
          } else {  // nested or non-numeric element: parse and drop
            ParseAttrValue();
            a.elems.push_back(Scalar{});
            non_numeric_array_ = true;
          }
        } while (lx_.Accept(","));
        lx_.Expect("]");
      }
    } else if (lx_.PeekIs("dense")) {
      lx_.Expect("dense");
      lx_.Expect("<");
      std::vector<Scalar> elems;
      bool any_float = false;
      auto one = [&]() {
        bool f;
        if (lx_.PeekIs("true") || lx_.PeekIs("false")) {
          Scalar s; s.i = lx_.Accept("true") ? 1 : (lx_.Expect("false"), 0); s.f = (double)s.i;
          elems.push_back(s);
          return;
        }
        const std::string n = lx_.Number(&f);
        Scalar s;
        s.is_float = f;
        if (f) { s.f = std::strtod(n.c_str(), nullptr); s.i = (int64_t)s.f; any_float = true; }
        else { s.i = std::strtoll(n.c_str(), nullptr, 0); s.f = (double)s.i; }
        elems.push_back(s);
      };
      bool splat = true;
      // dense<[[0, 0], [1, 1]]> : tensor<2x2xi64>: nested lists are flattened in row-major order
      std::function<void()> list = [&]() {
        if (lx_.Accept("]")) return;
        do {
          if (lx_.Accept("[")) list(); else one();
        } while (lx_.Accept(","));
        lx_.Expect("]");
      };
      if (lx_.Accept("[")) {
        splat = false;
        list();
      } else {
        one();
      }
      lx_.Expect(">");
      lx_.Expect(":");
      // tensor<NxT>: a splat is expanded to N elements
      lx_.Expect("tensor");
      lx_.Expect("<");
      int64_t n = 1;
      while (std::isdigit((unsigned char)lx_.Peek())) {
        n *= lx_.Digits();
        lx_.Expect("x");
      }
      const std::string et = lx_.Ident();
      lx_.Expect(">");
      if (splat && !elems.empty()) elems.assign((size_t)n, elems[0]);
      a.kind = (any_float || et[0] == 'f' || et == "bf16") ? Attr::DenseFloat : Attr::DenseInt;
      a.elems = std::move(elems);
    } else if (lx_.PeekIs("true") || lx_.PeekIs("false")) {
      a.kind = Attr::Bool;
      a.b = lx_.Accept("true");
      if (!a.b) lx_.Expect("false");
    } else if (lx_.PeekIs("unit")) {
      lx_.Expect("unit");
      a.kind = Attr::Unit;
    } else if (c == '-' || c == '+' || std::isdigit((unsigned char)c)) {
      const Scalar s = ParseNumberWithType();
      a.kind = s.is_float ? Attr::Float : Attr::Int;
      a.i = s.i;
      a.f = s.f;
    } else if (c == '{') {
      ParseAttrDict();  // nested dictionary: not interpreted
      a.kind = Attr::Unit;
    } else {
      // a type attribute or an affine map etc.: skip a bare identifier with optional <...>
      a.kind = Attr::String;
      a.s = lx_.Ident();
      if (lx_.Peek() == '<') lx_.SkipAngle();
    }
    return a;
  }

  std::map<std::string, Attr> ParseAttrDict() {
    std::map<std::string, Attr> d;
    lx_.Expect("{");
    if (lx_.Accept("}")) return d;
    do {
      const std::string name = lx_.Peek() == '"' ? lx_.String() : lx_.Ident();
      Attr a;
      if (lx_.Accept("=")) a = ParseAttrValue();
      d[name] = std::move(a);
    } while (lx_.Accept(","));
    lx_.Expect("}");
    return d;
  }

  int Lookup(const std::string &name) {
    auto it = by_name_.find(name);
    if (it == by_name_.end()) lx_.Fail("use of undefined value " + name);
    return it->second;
  }
  int Define(const std::string &name, const MemRefType &t) {
    if (by_name_.count(name)) lx_.Fail("redefinition of " + name);
    Value v;
    v.name = name;
    v.type = t;
    h_->values.push_back(v);
    by_name_[name] = (int)h_->values.size() - 1;
    return by_name_[name];
  }

  void ParseFunc() {
    lx_.Expect("func.func");
    lx_.Accept("private");
    lx_.Expect("@");
    h_->entry_name = lx_.Ident();
    lx_.Expect("(");
    if (!lx_.Accept(")")) {
      do {
        const std::string name = lx_.ValueName();
        lx_.Expect(":");
        const MemRefType t = ParseMemRef();
        const int id = Define(name, t);
        h_->values[id].arg_index = (int)h_->args.size();
        EntryArg ea;
        ea.value = id;
        if (lx_.Peek() == '{') {
          auto d = ParseAttrDict();
          if (d.count("byre.argname")) ea.argname = d["byre.argname"].s;
          if (d.count("byre.argtype")) ea.argtype = (int)d["byre.argtype"].i;
        }
        h_->args.push_back(ea);
      } while (lx_.Accept(","));
      lx_.Expect(")");
    }
    if (lx_.Accept("->")) lx_.Fail("entry functions return nothing in ByRE");
    if (lx_.Accept("attributes")) h_->func_attrs = ParseAttrDict();
    if (!h_->func_attrs.count("byre.entry_point")) lx_.Fail("function is not a byre.entry_point");
    lx_.Expect("{");
    while (!lx_.PeekIs("}")) ParseStmt();
    lx_.Expect("}");
  }

  std::vector<int> ParseOperands() {
    std::vector<int> ops;
    lx_.Expect("(");
    if (!lx_.Accept(")")) {
      do ops.push_back(Lookup(lx_.ValueName())); while (lx_.Accept(","));
      lx_.Expect(")");
    }
    return ops;
  }

  void ParseStmt() {
    const int line = lx_.line();
    if (lx_.Accept("return")) return;
    std::string result;
    if (lx_.Peek() == '%') {
      result = lx_.ValueName();
      lx_.Expect("=");
    }
    if (lx_.Accept("memref.alloc")) {
      lx_.Expect("(");
      lx_.Expect(")");
      if (lx_.Peek() == '{') ParseAttrDict();
      lx_.Expect(":");
      const MemRefType t = ParseMemRef();
      if (result.empty()) lx_.Fail("memref.alloc needs a result");
      const int id = Define(result, t);
      h_->values[id].is_alloc = true;
      return;
    }
    if (lx_.Accept("byre.compute")) {  // custom assembly
      Op op;
      op.name = "byre.compute";
      op.line = line;
      lx_.Expect("@");
      op.key = lx_.Peek() == '"' ? lx_.String() : lx_.Ident();
      op.operands = ParseOperands();
      if (lx_.Peek() == '{') op.attrs = ParseAttrDict();
      lx_.Expect(":");
      for (size_t i = 0; i < op.operands.size(); ++i) {
        if (i) lx_.Expect(",");
        CheckType(op.operands[i], ParseMemRef());
      }
      h_->ops.push_back(std::move(op));
      return;
    }
    if (lx_.Accept("byre.copy")) {  // byre.copy(%src, %dst) {callee = "cuda2cuda"} : type, type (ByreOps.td:170-186)
      Op op;
      op.name = "byre.copy";
      op.line = line;
      op.operands = ParseOperands();
      if (op.operands.size() != 2) lx_.Fail("byre.copy takes a source and a target");
      if (lx_.Peek() == '{') op.attrs = ParseAttrDict();
      lx_.Expect(":");
      CheckType(op.operands[0], ParseMemRef());
      lx_.Expect(",");
      CheckType(op.operands[1], ParseMemRef());
      // the registry key of a copy is its callee attribute (ByreInterface::getCalleeName, ByreBase.td:170-190)
      if (!op.attrs.count("callee") || op.attrs["callee"].s.empty()) lx_.Fail("byre.copy without callee");
      op.key = op.attrs["callee"].s;
      h_->ops.push_back(std::move(op));
      return;
    }
    if (lx_.Peek() == '"') {  // generic form
      Op op;
      op.name = lx_.String();
      op.line = line;
      op.operands = ParseOperands();
      if (lx_.Accept("<")) {  // inherent attributes printed as properties: "op"(...) <{offset = 0 : i64}> {device = "cuda"}
        op.attrs = ParseAttrDict();
        lx_.Expect(">");
      }
      if (lx_.Peek() == '{') {
        auto more = ParseAttrDict();
        for (auto &kv : more) op.attrs[kv.first] = std::move(kv.second);
      }
      lx_.Expect(":");
      lx_.Expect("(");
      for (size_t i = 0; i < op.operands.size(); ++i) {
        if (i) lx_.Expect(",");
        CheckType(op.operands[i], ParseMemRef());
      }
      lx_.Expect(")");
      lx_.Expect("->");
      if (op.name == "byre.alias") {
        const MemRefType rt = ParseMemRef();
        if (result.empty() || op.operands.size() != 1) lx_.Fail("byre.alias takes one operand and has one result");
        const int id = Define(result, rt);
        h_->values[id].alias_of = op.operands[0];
        h_->values[id].alias_offset = op.attrs.count("offset") ? op.attrs["offset"].i : 0;
        return;
      }
      if (lx_.Accept("(")) lx_.Expect(")");
      else lx_.Fail("ops with results are not supported: " + op.name);
      if (op.name == "byre.custom") {
        op.key = "custom";  // the registry key of every byre.custom (ByreDialect.cpp:538)
      } else if (op.name == "byre.compute") {
        if (!op.attrs.count("callee")) lx_.Fail("byre.compute without callee");
        op.key = op.attrs["callee"].s;
      } else {
        lx_.Fail("unsupported op " + op.name);
      }
      h_->ops.push_back(std::move(op));
      return;
    }
    lx_.Fail("unsupported statement");
  }

  void CheckType(int value, const MemRefType &t) {
    const MemRefType &d = h_->values[value].type;
    if (d.shape != t.shape || d.dtype != t.dtype || d.space != t.space)
      lx_.Fail("operand type does not match the definition of " + h_->values[value].name);
  }

  Lexer lx_;
  ByREHandle *h_;
  std::unordered_map<std::string, int> by_name_;
  bool non_numeric_array_ = false;
};

}  // namespace

common::Status ByREHandle::LoadFromText(const std::string &text) {
  entry_name.clear(); values.clear(); args.clear(); ops.clear(); func_attrs.clear();
  try {
    Parser(text, this).Run();
  } catch (const ParseError &e) {
    return common::Status::Fail(std::string("ByRE parse error: ") + e.what());
  }
  return common::Status::OK();
}

common::Status ByREHandle::LoadFromFile(const std::string &path) {
  std::ifstream f(path);
  if (!f) return common::Status::Fail("cannot open " + path);
  std::stringstream ss;
  ss << f.rdbuf();
  return LoadFromText(ss.str());
}

}  // namespace ir
}  // namespace brt
