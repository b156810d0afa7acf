// MLIR text -> fused-region program (see mlir_translate.h for what is
// recognised and which reference passes each piece stands in for).
//
// Structure: a character-level reader for the textual IR of the supported
// subset, and a symbolic evaluation of the function body in which every tensor
// value is "an expression of its own index space over reads of the function
// arguments".  Inlining a producer into a consumer is then substitution of
// index expressions through the consumer's affine map; the returned value's
// expression is emitted as the postfix program of one segment (one per
// operand of a trailing tensor.concat).
#include "mlir_translate.h"

#include <cmath>
#include <cstring>
#include <map>
#include <memory>
#include <stdexcept>

namespace afir_target {

using afir_region::ElemType;
using afir_region::OpCode;
using afir_region::Ref;

namespace {

struct Failure : std::runtime_error {
  using std::runtime_error::runtime_error;
};

// ------------------------------------------------------------ expressions ----

struct Index {
  enum Kind { Dim, Const, Gather } kind = Dim;
  int dim = 0;        // Dim / Gather: dim of the enclosing index space
  int64_t c = 0;      // Const
  int indexArg = -1;  // Gather: function argument holding the indices
};

struct Expr;
using ExprP = std::shared_ptr<const Expr>;
struct Expr {
  // Reduced: the row sum a tail expression works on; ExtentConst: an extent as a number
  enum Kind { Input, Constant, Unary, Binary, Matmul, Reduced, ExtentConst } kind = Constant;
  Ref extent;               // ExtentConst
  ElemType extentType = ElemType::F32;   // ... rounded through this type (arith.sitofp ... to f16);
                                         // Unary Cast: the type the value is rounded to
  int arg = -1, arg2 = -1;
  bool transA = false, transB = false;   // Matmul: operand stored transposed
  std::vector<Index> idx;   // Input: one per dim of the argument
  std::vector<Ref> slice;   // Input: start offsets (empty = none)
  float value = 0.f;        // Constant; alpha of Leaky
  OpCode op = OpCode::Add;
  ExprP a, b;
};

struct Tensor {
  std::vector<Ref> shape;
  ElemType elem = ElemType::F32;
  ExprP expr;                      // null: tensor.empty
  bool filled = false;
  float fill = 0.f;
  bool reduced = false;            // expr is the summand over iterSizes
  ExprP tail;                      // reduced: what happens to the row's sum (an expression in Expr::Reduced), or null
  std::vector<Ref> iterSizes;
  std::vector<std::shared_ptr<Tensor>> parts;  // tensor.concat along dim 0
  int directArg = -1;
};
using TensorP = std::shared_ptr<Tensor>;

struct Value {
  // ExtentFloat: an extent converted to a float type (arith.sitofp of a cast tensor.dim)
  enum Kind { None, TensorV, Float, Int, Extent, ExtentFloat, IndexV, Scalar, Accumulator } kind = None;
  TensorP tensor;
  double number = 0.0;   // Float / Int
  ElemType elem = ElemType::F32;
  Ref extent;            // Extent
  Index index;           // IndexV
  ExprP scalar;          // Scalar (inside a generic body)
  int blockArgOperand = -1;  // body block argument of `ins` operand N (for index tensors)
};

struct AffineMap {
  int numDims = 0;
  std::vector<Index> results;  // Dim / Const only
  bool isIdentity() const {
    if ((int)results.size() != numDims) return false;
    for (int i = 0; i < numDims; ++i)
      if (results[i].kind != Index::Dim || results[i].dim != i) return false;
    return true;
  }
};

// float -> f16 / bf16 -> float, round to nearest even: a constant written
// `0.1 : f16` has the value of the f16 nearest to 0.1
float roundThroughF16(float f) {
  uint32_t x;
  std::memcpy(&x, &f, 4);
  const uint32_t sign = x & 0x80000000u;
  x &= 0x7fffffffu;
  if (x >= 0x7f800000u) return f;                       // inf / nan
  if (x >= 0x477ff000u) {                               // rounds to >= 65520: inf
    uint32_t inf = sign | 0x7f800000u;
    std::memcpy(&f, &inf, 4);
    return f;
  }
  if (x < 0x38800000u) {                                // f16 subnormal range: quantum 2^-24
    float a;
    std::memcpy(&a, &x, 4);
    float q = std::nearbyintf(a * 16777216.0f) / 16777216.0f;
    return sign ? -q : q;
  }
  x += 0xfffu + ((x >> 13) & 1u);
  x &= ~0x1fffu;
  x |= sign;
  std::memcpy(&f, &x, 4);
  return f;
}
float roundThroughBf16(float f) {
  uint32_t x;
  std::memcpy(&x, &f, 4);
  if ((x & 0x7fffffffu) > 0x7f800000u) return f;
  x += 0x7fffu + ((x >> 16) & 1u);
  x &= 0xffff0000u;
  std::memcpy(&f, &x, 4);
  return f;
}

ExprP makeConst(float v) {
  auto e = std::make_shared<Expr>();
  e->kind = Expr::Constant;
  e->value = v;
  return e;
}
ExprP makeUnary(OpCode op, ExprP a, float alpha = 0.f) {
  auto e = std::make_shared<Expr>();
  e->kind = Expr::Unary;
  e->op = op;
  e->a = std::move(a);
  e->value = alpha;
  return e;
}
// x rounded to `type` and widened again (arith.truncf + arith.extf, afir.cast); float32 keeps x
ExprP makeCast(ElemType type, ExprP a) {
  if (type == ElemType::F32) return a;
  if (a->kind == Expr::Unary && a->op == OpCode::Cast && a->extentType == type) return a;
  auto e = std::make_shared<Expr>();
  e->kind = Expr::Unary;
  e->op = OpCode::Cast;
  e->extentType = type;
  e->a = std::move(a);
  return e;
}
// the same unary node over another operand
ExprP withOperand(const ExprP &unary, ExprP a) {
  auto e = std::make_shared<Expr>(*unary);
  e->a = std::move(a);
  return e;
}
bool isConst(const ExprP &e, float v) { return e->kind == Expr::Constant && e->value == v && !std::signbit(e->value); }

ExprP makeBinary(OpCode op, ExprP a, ExprP b) {
  // relu and leaky relu as the reference spells them (maximumf(x, 0),
  // maximumf(x, mulf(x, alpha)); ComputeConversion.cpp:718-726,
  // examples/matmul-add-leakyrelu/step0_input.mlir:40-52)
  if (op == OpCode::Max) {
    if (isConst(b, 0.f)) return makeUnary(OpCode::Relu, a);
    if (isConst(a, 0.f)) return makeUnary(OpCode::Relu, b);
    auto scaled = [](const ExprP &x, const ExprP &m, float *alpha) {
      if (m->kind != Expr::Binary || m->op != OpCode::Mul) return false;
      if (m->a == x && m->b->kind == Expr::Constant) { *alpha = m->b->value; return true; }
      if (m->b == x && m->a->kind == Expr::Constant) { *alpha = m->a->value; return true; }
      return false;
    };
    float alpha;
    if (scaled(a, b, &alpha)) return makeUnary(OpCode::Leaky, a, alpha);
    if (scaled(b, a, &alpha)) return makeUnary(OpCode::Leaky, b, alpha);
  }
  auto e = std::make_shared<Expr>();
  e->kind = Expr::Binary;
  e->op = op;
  e->a = std::move(a);
  e->b = std::move(b);
  return e;
}

// e is defined over some index space; `with` gives, for every dim of that
// space, its expression in the new space.
ExprP substitute(const ExprP &e, const std::vector<Index> &with) {
  switch (e->kind) {
    case Expr::Constant: case Expr::Reduced: case Expr::ExtentConst: return e;
    case Expr::Matmul: {
      for (size_t i = 0; i < with.size(); ++i)
        if (with[i].kind != Index::Dim || with[i].dim != (int)i)
          throw Failure("a matmul result can only be consumed through identity maps");
      return e;
    }
    case Expr::Unary: return withOperand(e, substitute(e->a, with));
    case Expr::Binary: {
      auto r = std::make_shared<Expr>(*e);
      r->a = substitute(e->a, with);
      r->b = substitute(e->b, with);
      return r;
    }
    case Expr::Input: {
      auto r = std::make_shared<Expr>(*e);
      int gathers = 0;
      for (Index &ix : r->idx) {
        if (ix.kind == Index::Const) continue;
        if (ix.dim < 0 || ix.dim >= (int)with.size()) throw Failure("affine map refers to a missing dimension");
        const Index &n = with[ix.dim];
        if (ix.kind == Index::Gather) {
          if (n.kind != Index::Dim) throw Failure("a gathered dimension can only be re-indexed by a plain dimension");
          ix.dim = n.dim;
        } else {
          ix = n;
        }
      }
      for (const Index &ix : r->idx) gathers += ix.kind == Index::Gather;
      if (gathers > 1) throw Failure("more than one gathered dimension in one read");
      return r;
    }
  }
  return e;
}

// value at (d + offsets) of every read
ExprP offsetReads(const ExprP &e, const std::vector<Ref> &offsets) {
  switch (e->kind) {
    case Expr::Constant: case Expr::ExtentConst: return e;
    case Expr::Reduced: throw Failure("extract_slice of a reduced value is not supported");
    case Expr::Matmul: throw Failure("extract_slice of a matmul result is not supported");
    case Expr::Unary: return withOperand(e, offsetReads(e->a, offsets));
    case Expr::Binary: {
      auto r = std::make_shared<Expr>(*e);
      r->a = offsetReads(e->a, offsets);
      r->b = offsetReads(e->b, offsets);
      return r;
    }
    case Expr::Input: {
      auto r = std::make_shared<Expr>(*e);
      if (r->slice.empty()) r->slice.assign(r->idx.size(), Ref::value(0));
      for (size_t d = 0; d < r->idx.size(); ++d) {
        const Index &ix = r->idx[d];
        if (ix.kind == Index::Const) continue;
        const Ref &o = offsets[ix.dim];
        if (o.arg < 0 && o.constant == 0) continue;
        Ref &cur = r->slice[d];
        if (cur.arg < 0 && o.arg < 0) cur = Ref::value(cur.constant + o.constant);
        else if (cur.arg < 0 && cur.constant == 0) cur = o;
        else throw Failure("nested extract_slice offsets that are not constants");
      }
      return r;
    }
  }
  return e;
}

// ------------------------------------------------------------------ reader ----

class Reader {
 public:
  explicit Reader(const std::string &text) : s_(text) {}

  [[noreturn]] void fail(const std::string &msg) const {
    int line = 1;
    for (size_t i = 0; i < pos_ && i < s_.size(); ++i) line += s_[i] == '\n';
    throw Failure("line " + std::to_string(line) + ": " + msg);
  }
  void skip() {
    for (;;) {
      while (pos_ < s_.size() && isspace((unsigned char)s_[pos_])) ++pos_;
      if (pos_ + 1 < s_.size() && s_[pos_] == '/' && s_[pos_ + 1] == '/') {
        while (pos_ < s_.size() && s_[pos_] != '\n') ++pos_;
        continue;
      }
      break;
    }
  }
  bool atEnd() { skip(); return pos_ >= s_.size(); }
  char peek() { skip(); return pos_ < s_.size() ? s_[pos_] : '\0'; }
  bool eat(char c) {
    if (peek() == c) { ++pos_; return true; }
    return false;
  }
  void expect(char c) {
    if (!eat(c)) fail(std::string("expected '") + c + "'");
  }
  bool eatArrow() {
    skip();
    if (s_.compare(pos_, 2, "->") == 0) { pos_ += 2; return true; }
    return false;
  }
  static bool identChar(char c) { return isalnum((unsigned char)c) || c == '_' || c == '.' || c == '$'; }
  std::string peekIdent() {
    skip();
    size_t p = pos_;
    while (p < s_.size() && identChar(s_[p])) ++p;
    return s_.substr(pos_, p - pos_);
  }
  std::string ident() {
    std::string id = peekIdent();
    if (id.empty()) fail("expected an identifier");
    pos_ += id.size();
    return id;
  }
  bool eatWord(const char *w) {
    if (peekIdent() == w) { pos_ += std::strlen(w); return true; }
    return false;
  }
  std::string sigil(char c, const char *what) {  // %name, @name, #name, ^name
    skip();
    if (pos_ >= s_.size() || s_[pos_] != c) fail(std::string("expected ") + what);
    size_t p = pos_ + 1;
    while (p < s_.size() && (identChar(s_[p]) || s_[p] == '#' || s_[p] == '-')) {
      if (s_[p] == '-' && p + 1 < s_.size() && s_[p + 1] == '>') break;
      ++p;
    }
    std::string r = s_.substr(pos_, p - pos_);
    pos_ = p;
    return r;
  }
  std::string ssa() { return sigil('%', "an SSA value (%name)"); }
  bool peekNumber() {
    char c = peek();
    return isdigit((unsigned char)c) || c == '-' || c == '+';
  }
  double number(bool *isInt = nullptr) {
    skip();
    size_t p = pos_;
    if (p < s_.size() && (s_[p] == '-' || s_[p] == '+')) ++p;
    bool digits = false, integer = true;
    while (p < s_.size() && isdigit((unsigned char)s_[p])) { ++p; digits = true; }
    if (p < s_.size() && s_[p] == '.') {
      integer = false;
      ++p;
      while (p < s_.size() && isdigit((unsigned char)s_[p])) { ++p; digits = true; }
    }
    if (digits && p < s_.size() && (s_[p] == 'e' || s_[p] == 'E')) {
      size_t q = p + 1;
      if (q < s_.size() && (s_[q] == '-' || s_[q] == '+')) ++q;
      if (q < s_.size() && isdigit((unsigned char)s_[q])) {
        integer = false;
        while (q < s_.size() && isdigit((unsigned char)s_[q])) ++q;
        p = q;
      }
    }
    if (!digits) fail("expected a number");
    double v = std::strtod(s_.substr(pos_, p - pos_).c_str(), nullptr);
    pos_ = p;
    if (isInt) *isInt = integer;
    return v;
  }
  int64_t integer() {
    bool isInt = false;
    double v = number(&isInt);
    if (!isInt) fail("expected an integer");
    return (int64_t)v;
  }
  // Skips one balanced attribute value / dictionary / type list.
  void skipBalanced() {
    skip();
    int depth = 0;
    while (pos_ < s_.size()) {
      char c = s_[pos_];
      if (c == '"') {
        ++pos_;
        while (pos_ < s_.size() && s_[pos_] != '"') pos_ += (s_[pos_] == '\\') ? 2 : 1;
        ++pos_;
        continue;
      }
      if (c == '-' && pos_ + 1 < s_.size() && s_[pos_ + 1] == '>') { pos_ += 2; continue; }
      if (c == '{' || c == '[' || c == '(' || c == '<') ++depth;
      else if (c == '}' || c == ']' || c == ')' || c == '>') {
        if (depth == 0) return;
        --depth;
        if (depth == 0) { ++pos_; skip();
          // a value such as `#afir.x<...>` or `dense<...> : type` may continue
          if (pos_ < s_.size() && (s_[pos_] == ',' || s_[pos_] == '}' || s_[pos_] == ']' || s_[pos_] == ')')) return;
          continue; }
      } else if ((c == ',') && depth == 0) {
        return;
      }
      ++pos_;
    }
  }

 private:
  const std::string &s_;
  size_t pos_ = 0;
};

struct TypeInfo {
  bool isTensor = false;
  std::vector<int64_t> shape;  // -1 = dynamic
  std::string elemName;
  ElemType elem = ElemType::F32;
  bool elemKnown = false;
};

bool elemFromName(const std::string &n, ElemType *t) {
  if (n == "f16") { *t = ElemType::F16; return true; }
  if (n == "bf16") { *t = ElemType::BF16; return true; }
  if (n == "f32") { *t = ElemType::F32; return true; }
  if (n == "i32") { *t = ElemType::I32; return true; }
  if (n == "i64") { *t = ElemType::I64; return true; }
  if (n == "i16") { *t = ElemType::I16; return true; }
  return false;
}

// ------------------------------------------------------------- translator ----

class Translator {
 public:
  explicit Translator(const std::string &text) : r_(text) {}

  void run(Translation *out) {
    while (!r_.atEnd()) {
      char c = r_.peek();
      if (c == '#') {
        parseAlias();
      } else if (r_.eatWord("module")) {
        if (r_.peek() == '@') r_.sigil('@', "a symbol");
        if (r_.eatWord("attributes")) { r_.expect('{'); skipDict(); }
        r_.expect('{');
        inModule_ = true;
      } else if (r_.peekIdent() == "func.func") {
        parseFunction(out);
        return;
      } else if (c == '}' && inModule_) {
        r_.eat('}');
        inModule_ = false;
      } else {
        r_.fail("expected an affine map alias, 'module' or 'func.func'");
      }
    }
    r_.fail("no func.func found");
  }

 private:
  // `{` has been consumed: skip to the matching `}`
  void skipDict() {
    for (;;) {
      r_.skipBalanced();
      if (r_.eat('}')) return;
      if (!r_.eat(',')) r_.fail("malformed attribute dictionary");
    }
  }

  AffineMap parseAffineMapBody() {  // after "affine_map"
    AffineMap m;
    r_.expect('<');
    r_.expect('(');
    std::vector<std::string> dims;
    if (!r_.eat(')')) {
      do dims.push_back(r_.ident()); while (r_.eat(','));
      r_.expect(')');
    }
    if (r_.peek() == '[') r_.fail("affine maps with symbols are not supported");
    if (!r_.eatArrow()) r_.fail("expected '->' in affine_map");
    r_.expect('(');
    m.numDims = (int)dims.size();
    if (!r_.eat(')')) {
      do {
        Index ix;
        if (r_.peekNumber()) {
          ix.kind = Index::Const;
          ix.c = r_.integer();
        } else {
          std::string d = r_.ident();
          ix.kind = Index::Dim;
          ix.dim = -1;
          for (size_t i = 0; i < dims.size(); ++i)
            if (dims[i] == d) ix.dim = (int)i;
          if (ix.dim < 0) r_.fail("unknown dimension '" + d + "' in affine_map");
        }
        char c = r_.peek();
        if (c != ',' && c != ')')
          r_.fail("only dimensions and constants are supported as affine map results");
        m.results.push_back(ix);
      } while (r_.eat(','));
      r_.expect(')');
    }
    r_.expect('>');
    return m;
  }

  void parseAlias() {
    std::string name = r_.sigil('#', "an attribute alias");
    r_.expect('=');
    if (r_.eatWord("affine_map")) {
      aliases_[name] = parseAffineMapBody();
    } else {
      r_.skipBalanced();  // some other attribute alias: not needed
    }
  }

  AffineMap parseMapRef() {
    if (r_.peek() == '#') {
      std::string name = r_.sigil('#', "an attribute alias");
      auto it = aliases_.find(name);
      if (it == aliases_.end()) r_.fail("unknown affine map alias " + name);
      return it->second;
    }
    if (!r_.eatWord("affine_map")) r_.fail("expected an affine map");
    return parseAffineMapBody();
  }

  TypeInfo parseType() {
    TypeInfo t;
    std::string id = r_.ident();
    if (id == "tensor") {
      t.isTensor = true;
      r_.expect('<');
      for (;;) {
        char c = r_.peek();
        if (c == '?') {
          r_.eat('?');
          t.shape.push_back(-1);
          r_.expect('x');
        } else if (isdigit((unsigned char)c)) {
          t.shape.push_back(r_.integer());
          r_.expect('x');
        } else {
          t.elemName = r_.ident();
          break;
        }
      }
      if (r_.eat(',')) r_.skipBalanced();  // encoding attribute
      r_.expect('>');
    } else {
      t.elemName = id;
    }
    t.elemKnown = elemFromName(t.elemName, &t.elem);
    return t;
  }

  // ---- values ----
  Value &lookup(const std::string &name) {
    auto it = body_.find(name);
    if (it != body_.end()) return it->second;
    it = env_.find(name);
    if (it == env_.end()) r_.fail("use of undefined value " + name);
    return it->second;
  }
  TensorP tensorOf(const std::string &name) {
    Value &v = lookup(name);
    if (v.kind != Value::TensorV) r_.fail(name + " is not a tensor");
    return v.tensor;
  }
  Ref extentOf(const std::string &name) {
    Value &v = lookup(name);
    if (v.kind == Value::Extent) return v.extent;
    if (v.kind == Value::Int) return Ref::value((int64_t)v.number);
    r_.fail(name + " is not an extent (tensor.dim result or integer constant)");
  }
  void define(const std::string &name, Value v) { (inBody_ ? body_ : env_)[name] = std::move(v); }
  void defineTensor(const std::string &name, TensorP t) {
    Value v;
    v.kind = Value::TensorV;
    v.tensor = std::move(t);
    define(name, std::move(v));
  }

  // ---- function ----
  void parseFunction(Translation *out) {
    r_.eatWord("func.func");
    std::string vis = r_.peekIdent();
    if (vis == "private" || vis == "public") r_.ident();
    out->functionName = r_.sigil('@', "a function name").substr(1);
    r_.expect('(');
    if (!r_.eat(')')) {
      do {
        std::string name = r_.ssa();
        r_.expect(':');
        TypeInfo t = parseType();
        if (r_.peek() == '{') { r_.eat('{'); skipDict(); }
        if (!t.isTensor) r_.fail("function argument " + name + " is not a tensor");
        if (!t.elemKnown) r_.fail("unsupported element type '" + t.elemName + "' of argument " + name);
        if ((int)t.shape.size() > afir_region::kMaxRank) r_.fail("argument " + name + " has rank > 3");
        const int argIndex = (int)args_.size();
        afir_region::Arg a;
        a.type = t.elem;
        a.rank = (int)t.shape.size();
        args_.push_back(a);
        auto tv = std::make_shared<Tensor>();
        tv->elem = t.elem;
        tv->directArg = argIndex;
        for (size_t d = 0; d < t.shape.size(); ++d) tv->shape.push_back(Ref::dimOf(argIndex, (int)d));
        // i16 / i32 tensors are values to the afir integer ops (and i32 an index
        // tensor to linalg.generic); i64 is an index type only
        if (afir_region::isFloat(t.elem) || afir_region::isRegionInt(t.elem)) {
          auto e = std::make_shared<Expr>();
          e->kind = Expr::Input;
          e->arg = argIndex;
          for (size_t d = 0; d < t.shape.size(); ++d) {
            Index ix;
            ix.dim = (int)d;
            e->idx.push_back(ix);
          }
          tv->expr = e;
        }
        defineTensor(name, tv);
      } while (r_.eat(','));
      r_.expect(')');
    }
    if (r_.eatArrow()) {
      if (r_.eat('(')) {
        do parseType(); while (r_.eat(','));
        r_.expect(')');
      } else {
        parseType();
      }
    }
    if (r_.eatWord("attributes")) { r_.expect('{'); skipDict(); }
    r_.expect('{');
    TensorP result;
    while (!result) {
      if (r_.peek() == '}') r_.fail("function has no return");
      try {
        result = parseOperation();
      } catch (const Failure &f) {
        if (std::strncmp(f.what(), "line ", 5) == 0) throw;
        r_.fail(f.what());  // adds the position
      }
    }
    emit(result, out);
  }

  // Parses one operation of the function body; returns the returned tensor
  // when the operation is the return.
  TensorP parseOperation() {
    std::vector<std::string> results;
    if (r_.peek() == '%') {
      do results.push_back(r_.ssa()); while (r_.eat(','));
      r_.expect('=');
    }
    const std::string op = r_.ident();
    auto one = [&]() -> const std::string & {
      if (results.size() != 1) r_.fail(op + " defines exactly one value");
      return results[0];
    };
    if (op == "return" || op == "func.return") {
      std::vector<std::string> vals;
      if (r_.peek() == '%') {
        do vals.push_back(r_.ssa()); while (r_.eat(','));
        r_.expect(':');
        do parseType(); while (r_.eat(','));
      }
      if (vals.size() != 1) r_.fail("functions returning exactly one tensor are supported");
      return tensorOf(vals[0]);
    }
    if (op == "arith.constant") {
      parseConstant(one());
    } else if (op == "tensor.dim") {
      std::string t = r_.ssa();
      r_.expect(',');
      std::string c = r_.ssa();
      r_.expect(':');
      parseType();
      Value &cv = lookup(c);
      if (cv.kind != Value::Int) r_.fail("tensor.dim needs a constant dimension index");
      TensorP tv = tensorOf(t);
      if (cv.number < 0 || cv.number >= (double)tv->shape.size()) r_.fail("tensor.dim index out of range");
      Value v;
      v.kind = Value::Extent;
      v.extent = tv->shape[(size_t)cv.number];
      define(one(), v);
    } else if (op == "arith.index_cast" || op == "arith.sitofp" || op == "arith.uitofp") {
      // an extent as a number, outside any generic: index -> iN -> float (mean = sum / N,
      // examples/broadcast-add-reduce/step0_input_mean.mlir:73-74)
      Value &src = lookup(r_.ssa());
      r_.expect(':');
      parseType();
      if (!r_.eatWord("to")) r_.fail("expected 'to' in " + op);
      TypeInfo to = parseType();
      Value v;
      if (op == "arith.index_cast") {
        if (src.kind != Value::Extent && src.kind != Value::Int) r_.fail("arith.index_cast of a value that is not an extent");
        v = src;
      } else if (src.kind == Value::Int) {
        v.kind = Value::Float;
        float f = (float)src.number;
        if (to.elemName == "f16") f = roundThroughF16(f);
        else if (to.elemName == "bf16") f = roundThroughBf16(f);
        else if (to.elemName != "f32") r_.fail("unsupported float type " + to.elemName);
        v.number = f;
        v.scalar = makeConst(f);
      } else {
        if (src.kind != Value::Extent) r_.fail(op + " of a value that is not an extent");
        if (src.extent.arg < 0) r_.fail(op + ": internal error, constant extent");
        v.kind = Value::ExtentFloat;
        v.extent = src.extent;
        if (to.elemName == "f16") v.elem = ElemType::F16;
        else if (to.elemName == "bf16") v.elem = ElemType::BF16;
        else if (to.elemName == "f32") v.elem = ElemType::F32;
        else r_.fail("unsupported float type " + to.elemName);
      }
      define(one(), v);
    } else if (op == "tensor.empty") {
      r_.expect('(');
      std::vector<Ref> dyn;
      if (!r_.eat(')')) {
        do dyn.push_back(extentOf(r_.ssa())); while (r_.eat(','));
        r_.expect(')');
      }
      r_.expect(':');
      TypeInfo t = parseType();
      auto tv = std::make_shared<Tensor>();
      tv->elem = t.elem;
      size_t at = 0;
      for (int64_t d : t.shape) {
        if (d >= 0) tv->shape.push_back(Ref::value(d));
        else if (at < dyn.size()) tv->shape.push_back(dyn[at++]);
        else r_.fail("tensor.empty: too few dynamic extents");
      }
      defineTensor(one(), tv);
    } else if (op == "linalg.fill") {
      parseFill(one());
    } else if (op == "linalg.generic") {
      parseGeneric(results);
    } else if (op == "linalg.matmul") {
      parseMatmul(one(), op, false, false, false);
    } else if (op == "linalg.matmul_transpose_a") {
      parseMatmul(one(), op, true, false, false);
    } else if (op == "linalg.matmul_transpose_b") {
      parseMatmul(one(), op, false, true, false);
    } else if (op == "linalg.batch_matmul") {
      parseMatmul(one(), op, false, false, true);
    } else if (op == "linalg.batch_matmul_transpose_a") {
      parseMatmul(one(), op, true, false, true);
    } else if (op == "linalg.batch_matmul_transpose_b") {
      parseMatmul(one(), op, false, true, true);
    } else if (op == "linalg.elementwise") {
      parseElementwise(one());
    } else if (op == "linalg.transpose") {
      parseTranspose(one());
    } else if (op == "linalg.reduce") {
      parseReduce(one());
    } else if (op == "linalg.broadcast") {
      parseBroadcast(one());
    } else if (op == "tensor.collapse_shape" || op == "tensor.expand_shape") {
      parseReshape(one(), op == "tensor.expand_shape");
    } else if (namedElementwise(op.compare(0, 7, "linalg.") == 0 ? op.substr(7) : std::string(), nullptr, nullptr)) {
      parseNamedElementwise(one(), op.substr(7));
    } else if (op == "tensor.extract_slice") {
      parseExtractSlice(one());
    } else if (op == "tensor.concat") {
      parseConcat(one());
    } else if (op.compare(0, 5, "afir.") == 0) {
      parseAfir(op.substr(5), one());
    } else {
      r_.fail("operation '" + op + "' has no HIP lowering");
    }
    return nullptr;
  }

  void parseConstant(const std::string &result) {
    Value v;
    if (r_.eatWord("true") || r_.eatWord("false")) r_.fail("boolean constants are not supported");
    if (r_.peekIdent() == "dense") {
      // dense<c> : tensor<...>: a tensor of one value (what linalg ops take as an init)
      r_.ident();
      r_.expect('<');
      if (r_.peek() == '[') r_.fail("dense constants other than splats (dense<c>) are not supported");
      const double c = r_.number();
      r_.expect('>');
      r_.expect(':');
      TypeInfo t = parseType();
      if (!t.isTensor || !t.elemKnown || !afir_region::isFloat(t.elem)) r_.fail("a dense splat must be a float tensor");
      auto tv = std::make_shared<Tensor>();
      tv->elem = t.elem;
      for (int64_t d : t.shape) {
        if (d < 0) r_.fail("a dense constant has a static shape");
        tv->shape.push_back(Ref::value(d));
      }
      float f = (float)c;
      if (t.elem == ElemType::F16) f = roundThroughF16(f);
      else if (t.elem == ElemType::BF16) f = roundThroughBf16(f);
      tv->filled = true;
      tv->fill = f;
      tv->expr = makeConst(f);
      defineTensor(result, tv);
      return;
    }
    bool isInt = false;
    const double n = r_.number(&isInt);
    r_.expect(':');
    TypeInfo t = parseType();
    if (t.elemName == "index" || t.elemName[0] == 'i') {
      v.kind = Value::Int;
      v.number = n;
    } else {
      v.kind = Value::Float;
      float f = (float)n;
      if (t.elemName == "f16") f = roundThroughF16(f);
      else if (t.elemName == "bf16") f = roundThroughBf16(f);
      else if (t.elemName != "f32") r_.fail("unsupported constant type " + t.elemName);
      v.number = f;
      v.scalar = makeConst(f);
    }
    define(result, v);
  }

  struct Operands {
    std::vector<std::string> names;
    std::vector<TypeInfo> types;
  };
  Operands parseOperandGroup(const char *keyword) {  // ins(%a, %b : t, t)
    Operands o;
    if (!r_.eatWord(keyword)) return o;
    r_.expect('(');
    if (r_.eat(')')) return o;
    do o.names.push_back(r_.ssa()); while (r_.eat(','));
    r_.expect(':');
    do o.types.push_back(parseType()); while (r_.eat(','));
    r_.expect(')');
    if (o.names.size() != o.types.size()) r_.fail(std::string(keyword) + ": operand / type count mismatch");
    return o;
  }

  void parseFill(const std::string &result) {
    Operands ins = parseOperandGroup("ins"), outs = parseOperandGroup("outs");
    if (ins.names.size() != 1 || outs.names.size() != 1) r_.fail("linalg.fill needs one scalar and one tensor");
    if (r_.eatArrow()) parseType();
    Value &c = lookup(ins.names[0]);
    if (c.kind != Value::Float && c.kind != Value::Int) r_.fail("linalg.fill value must be a constant");
    TensorP init = tensorOf(outs.names[0]);
    auto tv = std::make_shared<Tensor>(*init);
    tv->directArg = -1;
    tv->filled = true;
    tv->fill = (float)c.number;
    tv->expr = makeConst((float)c.number);
    defineTensor(result, tv);
  }

  // linalg.matmul and its relatives: the matmul-like ops the reference's recogniser takes
  // (lib/Conversion/MarkStructuredOps/AnnotateMixMatmulSemanticsPass.cpp:244-256).
  //   matmul_transpose_a: A is [K, M]; matmul_transpose_b: B is [N, K];
  //   batch_matmul*: a leading batch dim on A, B and the result.
  void parseMatmul(const std::string &result, const std::string &op, bool ta, bool tb, bool batched) {
    if (r_.peek() == '{') { r_.eat('{'); skipDict(); }
    Operands ins = parseOperandGroup("ins"), outs = parseOperandGroup("outs");
    if (ins.names.size() != 2 || outs.names.size() != 1) r_.fail(op + " needs two inputs and one init");
    TypeInfo rt = outs.types[0];
    if (r_.eatArrow()) rt = parseType();
    TensorP a = tensorOf(ins.names[0]), b = tensorOf(ins.names[1]), init = tensorOf(outs.names[0]);
    const size_t rank = batched ? 3 : 2, b0 = batched ? 1 : 0;
    if (a->directArg < 0 || b->directArg < 0 || a->shape.size() != rank || b->shape.size() != rank)
      r_.fail(op + " operands must be rank-" + std::to_string(rank) + " function arguments");
    // The init is taken as zero: the reference's mix kernel overwrites C
    // (Matmul IterateAll, lib/Target/CannKernel/CannTranslation.cpp:1584-1628)
    // and its example passes an all-zero tensor.
    if (init->expr && !(init->directArg >= 0) && !(init->filled && init->fill == 0.f))
      r_.fail(op + " init must be a function argument, an empty tensor or a zero fill");
    auto e = std::make_shared<Expr>();
    e->kind = Expr::Matmul;
    e->arg = a->directArg;
    e->arg2 = b->directArg;
    e->transA = ta;
    e->transB = tb;
    auto tv = std::make_shared<Tensor>();
    tv->elem = rt.elemKnown ? rt.elem : init->elem;
    if (batched) tv->shape.push_back(a->shape[0]);
    tv->shape.push_back(a->shape[b0 + (ta ? 1 : 0)]);
    tv->shape.push_back(b->shape[b0 + (tb ? 0 : 1)]);
    tv->expr = e;
    defineTensor(result, tv);
  }

  // ---- named linalg ops (what the reference's --linalg-mark / --linalg-add-broadcast consume:
  // test/Dialect/AFIR/Transforms/linalgMark.mlir:35-44, linalgAddBroadcast.mlir:3-23) ----
  // the arithmetic of linalg.<name> / #linalg.elementwise_kind<name>: false for a kind this
  // backend has no lowering for (the transcendental functions)
  static bool namedElementwise(const std::string &name, OpCode *code, int *arity) {
    static const struct { const char *n; OpCode c; int arity; } table[] = {
        {"add", OpCode::Add, 2}, {"sub", OpCode::Sub, 2}, {"mul", OpCode::Mul, 2}, {"div", OpCode::Div, 2},
        {"max", OpCode::Max, 2}, {"min", OpCode::Min, 2}, {"max_signed", OpCode::Max, 2},
        {"min_signed", OpCode::Min, 2}, {"negf", OpCode::Neg, 1}, {"abs", OpCode::Neg, -1},
        // arities below -1 name a form built from the chain's own operations:
        // copy: x, square: x * x, reciprocal: 1 / x
        {"copy", OpCode::Add, -2}, {"square", OpCode::Mul, -3}, {"reciprocal", OpCode::Div, -4}};
    for (const auto &e : table)
      if (name == e.n) {
        if (code) *code = e.c;
        if (arity) *arity = e.arity;
        return true;
      }
    return false;
  }
  // result of an elementwise op over `ins` read through `maps` (one per input, then the output's)
  void defineElementwise(const std::string &result, const std::string &kind, const Operands &ins, const Operands &outs,
                         std::vector<AffineMap> maps) {
    OpCode code = OpCode::Add;
    int arity = 0;
    if (!namedElementwise(kind, &code, &arity)) r_.fail("elementwise kind '" + kind + "' has no HIP lowering");
    const int want = arity < 0 ? 1 : arity;
    if ((int)ins.names.size() != want || outs.names.size() != 1)
      r_.fail("elementwise '" + kind + "' takes " + std::to_string(want) + " input(s) and one init");
    TensorP outT = tensorOf(outs.names[0]);
    const int rank = (int)outT->shape.size();
    if (maps.empty()) {   // identity maps: operands of the output's shape
      AffineMap id;
      id.numDims = rank;
      for (int d = 0; d < rank; ++d) { Index ix; ix.dim = d; id.results.push_back(ix); }
      maps.assign(ins.names.size() + 1, id);
    }
    if (maps.size() != ins.names.size() + 1) r_.fail("elementwise: one indexing map per operand is required");
    if (!maps.back().isIdentity() || maps.back().numDims != rank) r_.fail("elementwise: the output map must be the identity");
    std::vector<ExprP> v;
    for (size_t i = 0; i < ins.names.size(); ++i) {
      TensorP t = tensorOf(ins.names[i]);
      if (!t->expr || t->reduced || !t->parts.empty() || !afir_region::isFloat(t->elem))
        r_.fail("elementwise: operand " + ins.names[i] + " is not an elementwise float value");
      if (maps[i].numDims != rank || maps[i].results.size() != t->shape.size())
        r_.fail("elementwise: the map of operand " + std::to_string(i) + " does not match its rank");
      v.push_back(substitute(t->expr, maps[i].results));
    }
    auto tv = std::make_shared<Tensor>();
    tv->elem = outT->elem;
    tv->shape = outT->shape;
    if (arity == 2) tv->expr = makeBinary(code, v[0], v[1]);
    else if (arity == 1) tv->expr = makeUnary(code, v[0]);
    else if (arity == -2) tv->expr = v[0];
    else if (arity == -3) tv->expr = makeBinary(OpCode::Mul, v[0], v[0]);
    else if (arity == -4) tv->expr = makeBinary(OpCode::Div, makeConst(1.f), v[0]);
    else tv->expr = makeBinary(OpCode::Max, v[0], makeUnary(OpCode::Neg, v[0]));   // |x| = max(x, -x), exactly
    defineTensor(result, tv);
  }
  // linalg.elementwise kind=#linalg.elementwise_kind<add> [indexing_maps = [...]] ins(...) outs(...) [-> type]
  void parseElementwise(const std::string &result) {
    if (!r_.eatWord("kind")) r_.fail("expected 'kind=' in linalg.elementwise");
    r_.expect('=');
    r_.sigil('#', "an elementwise kind");
    r_.expect('<');
    const std::string kind = r_.ident();
    r_.expect('>');
    std::vector<AffineMap> maps;
    if (r_.eatWord("indexing_maps")) {
      r_.expect('=');
      r_.expect('[');
      do maps.push_back(parseMapRef()); while (r_.eat(','));
      r_.expect(']');
    }
    if (r_.peek() == '{') { r_.eat('{'); skipDict(); }
    Operands ins = parseOperandGroup("ins"), outs = parseOperandGroup("outs");
    if (r_.eatArrow()) parseType();
    defineElementwise(result, kind, ins, outs, maps);
  }
  // linalg.add / sub / mul / div / max / min / negf / abs ins(...) outs(...) [-> type]
  void parseNamedElementwise(const std::string &result, const std::string &kind) {
    if (r_.peek() == '{') { r_.eat('{'); skipDict(); }
    Operands ins = parseOperandGroup("ins"), outs = parseOperandGroup("outs");
    if (r_.eatArrow()) parseType();
    defineElementwise(result, kind, ins, outs, {});
  }
  std::vector<int64_t> parseIntList(const char *keyword) {
    if (!r_.eatWord(keyword)) r_.fail(std::string("expected '") + keyword + " = [...]'");
    r_.expect('=');
    std::vector<int64_t> v;
    r_.expect('[');
    if (!r_.eat(']')) {
      do v.push_back(r_.integer()); while (r_.eat(','));
      r_.expect(']');
    }
    return v;
  }
  TensorP elementwiseSource(const std::string &name, const char *what) {
    TensorP t = tensorOf(name);
    if (!t->expr || t->reduced || !t->parts.empty()) r_.fail(std::string(what) + " of a value that is not elementwise");
    return t;
  }
  // linalg.transpose ins(%a : t) outs(%b : t) permutation = [p0, p1, ...]: result dim i is input dim p_i
  void parseTranspose(const std::string &result) {
    Operands ins = parseOperandGroup("ins"), outs = parseOperandGroup("outs");
    if (ins.names.size() != 1 || outs.names.size() != 1) r_.fail("linalg.transpose takes one input and one init");
    const std::vector<int64_t> perm = parseIntList("permutation");
    if (r_.eatArrow()) parseType();
    TensorP in = elementwiseSource(ins.names[0], "linalg.transpose"), outT = tensorOf(outs.names[0]);
    const size_t rank = in->shape.size();
    if (perm.size() != rank || outT->shape.size() != rank) r_.fail("linalg.transpose: the permutation does not match the rank");
    std::vector<Index> with(rank);
    std::vector<bool> seen(rank, false);
    auto tv = std::make_shared<Tensor>();
    tv->elem = outT->elem;
    for (size_t i = 0; i < rank; ++i) {
      if (perm[i] < 0 || perm[i] >= (int64_t)rank || seen[(size_t)perm[i]]) r_.fail("linalg.transpose: not a permutation");
      seen[(size_t)perm[i]] = true;
      with[(size_t)perm[i]].dim = (int)i;
      tv->shape.push_back(in->shape[(size_t)perm[i]]);
    }
    tv->expr = substitute(in->expr, with);
    defineTensor(result, tv);
  }
  // linalg.reduce ins(%a : t) outs(%init : t') dimensions = [last] (%x: f32, %acc: f32) { addf; yield }
  // or the short form linalg.reduce { arith.addf } ins(...) outs(...) dimensions = [last]: the sum
  // over the innermost dim into a zero-filled init, the one reduction this backend lowers (the
  // reference lowers only sums: ComputeConversion.cpp:731-740)
  void parseReduce(const std::string &result) {
    bool sum = false;
    if (r_.peek() == '{') {   // short form: the combiner's name in braces
      r_.eat('{');
      sum = r_.ident() == "arith.addf";
      if (r_.peek() == '{') { r_.eat('{'); skipDict(); }
      r_.expect('}');
      if (!sum) r_.fail("linalg.reduce: only a sum (arith.addf) has a HIP lowering");
    }
    Operands ins = parseOperandGroup("ins"), outs = parseOperandGroup("outs");
    if (ins.names.size() != 1 || outs.names.size() != 1) r_.fail("linalg.reduce takes one input and one init");
    const std::vector<int64_t> dims = parseIntList("dimensions");
    if (r_.peek() == '(') {   // the combiner region: (%in: f32, %acc: f32) { %s = arith.addf %in, %acc : f32  linalg.yield %s : f32 }
      r_.eat('(');
      std::vector<std::string> args;
      do { args.push_back(r_.ssa()); r_.expect(':'); parseType(); } while (r_.eat(','));
      r_.expect(')');
      r_.expect('{');
      if (args.size() != 2) r_.fail("linalg.reduce: the combiner takes two scalars");
      const std::string value = r_.ssa();
      r_.expect('=');
      if (r_.ident() != "arith.addf") r_.fail("linalg.reduce: only a sum (arith.addf) has a HIP lowering");
      const std::string x = r_.ssa();
      r_.expect(',');
      const std::string y = r_.ssa();
      if (!((x == args[0] && y == args[1]) || (x == args[1] && y == args[0])))
        r_.fail("linalg.reduce: the combiner must add its two arguments");
      if (r_.eatWord("fastmath")) { r_.expect('<'); r_.skipBalanced(); r_.expect('>'); }
      r_.expect(':');
      parseType();
      if (r_.ident() != "linalg.yield" || r_.ssa() != value) r_.fail("linalg.reduce: the combiner must yield its sum");
      r_.expect(':');
      parseType();
      r_.expect('}');
      sum = true;
    }
    if (!sum) r_.fail("linalg.reduce needs a combiner");
    if (r_.eatArrow()) parseType();
    TensorP in = elementwiseSource(ins.names[0], "linalg.reduce"), outT = tensorOf(outs.names[0]);
    const size_t rank = in->shape.size();
    if (rank < 2 || dims.size() != 1 || dims[0] != (int64_t)rank - 1 || outT->shape.size() != rank - 1)
      r_.fail("linalg.reduce: only a reduction of the innermost dim of a tensor of rank 2 or 3 has a HIP lowering");
    if (!afir_region::isFloat(in->elem)) r_.fail("linalg.reduce: only float tensors");
    if (!(outT->filled && outT->fill == 0.f)) r_.fail("linalg.reduce needs a zero-filled init (linalg.fill 0)");
    auto tv = std::make_shared<Tensor>();
    tv->elem = outT->elem;
    tv->shape = outT->shape;
    tv->reduced = true;
    tv->expr = in->expr;
    tv->iterSizes = in->shape;
    defineTensor(result, tv);
  }
  // linalg.broadcast ins(%a : t) outs(%b : t) dimensions = [...]: the result dims that are added
  void parseBroadcast(const std::string &result) {
    Operands ins = parseOperandGroup("ins"), outs = parseOperandGroup("outs");
    if (ins.names.size() != 1 || outs.names.size() != 1) r_.fail("linalg.broadcast takes one input and one init");
    const std::vector<int64_t> added = parseIntList("dimensions");
    if (r_.eatArrow()) parseType();
    TensorP in = elementwiseSource(ins.names[0], "linalg.broadcast"), outT = tensorOf(outs.names[0]);
    const size_t rank = outT->shape.size();
    if (in->shape.size() + added.size() != rank) r_.fail("linalg.broadcast: input rank + added dims must be the result rank");
    std::vector<bool> isAdded(rank, false);
    for (int64_t d : added) {
      if (d < 0 || d >= (int64_t)rank || isAdded[(size_t)d]) r_.fail("linalg.broadcast: bad 'dimensions'");
      isAdded[(size_t)d] = true;
    }
    std::vector<Index> with;
    auto tv = std::make_shared<Tensor>();
    tv->elem = in->elem;
    size_t own = 0;
    for (size_t d = 0; d < rank; ++d) {
      if (isAdded[d]) {
        tv->shape.push_back(outT->shape[d]);
      } else {
        Index ix;
        ix.dim = (int)d;
        with.push_back(ix);
        tv->shape.push_back(in->shape[own++]);
      }
    }
    tv->expr = substitute(in->expr, with);
    defineTensor(result, tv);
  }
  // tensor.collapse_shape %x [[0, 1], [2]] : tensor<8x1x32xf32> into tensor<8x32xf32>
  // tensor.expand_shape %x [[0, 1], [2]] output_shape [8, 1, 32] : tensor<8x32xf32> into tensor<8x1x32xf32>
  // Supported where a reassociation group holds at most one dim whose (static) extent is not 1:
  // dims of extent 1 come and go, nothing is re-linearised.
  void parseReshape(const std::string &result, bool expand) {
    TensorP src = elementwiseSource(r_.ssa(), expand ? "tensor.expand_shape" : "tensor.collapse_shape");
    std::vector<std::vector<int64_t>> groups;
    r_.expect('[');
    if (!r_.eat(']')) {
      do {
        std::vector<int64_t> g;
        r_.expect('[');
        if (!r_.eat(']')) {
          do g.push_back(r_.integer()); while (r_.eat(','));
          r_.expect(']');
        }
        groups.push_back(g);
      } while (r_.eat(','));
      r_.expect(']');
    }
    if (r_.eatWord("output_shape")) (void)parseSliceList();   // [4, 1, %n]: the result type says the same
    r_.expect(':');
    TypeInfo from = parseType();
    if (!r_.eatWord("into")) r_.fail("expected 'into' in a reshape");
    TypeInfo to = parseType();
    const TypeInfo &wide = expand ? to : from, &narrow = expand ? from : to;   // wide: the side with more dims
    if (groups.size() != narrow.shape.size() || from.shape.size() != src->shape.size())
      r_.fail("reshape: the reassociation does not match the types");
    // per group: the one wide dim that is not a static 1 (-1: all are 1)
    std::vector<int> keep(groups.size(), -1);
    size_t expect = 0;
    for (size_t g = 0; g < groups.size(); ++g)
      for (int64_t d : groups[g]) {
        if (d != (int64_t)expect++ || d >= (int64_t)wide.shape.size()) r_.fail("reshape: reassociation indices must be 0, 1, 2, ... in order");
        if (wide.shape[(size_t)d] == 1) continue;
        if (keep[g] >= 0) r_.fail("reshapes that merge or split dims of extent other than 1 are not supported");
        keep[g] = (int)d;
      }
    if (expect != wide.shape.size()) r_.fail("reshape: the reassociation does not cover every dim");
    auto tv = std::make_shared<Tensor>();
    tv->elem = src->elem;
    std::vector<Index> with(src->shape.size());
    if (!expand) {
      // source = wide: its kept dim of group g is result dim g, the others are read at 0
      for (size_t g = 0; g < groups.size(); ++g) {
        for (int64_t d : groups[g]) {
          Index ix;
          if ((int)d == keep[g]) ix.dim = (int)g;
          else { ix.kind = Index::Const; ix.c = 0; }
          with[(size_t)d] = ix;
        }
        tv->shape.push_back(keep[g] >= 0 ? src->shape[(size_t)keep[g]] : Ref::value(1));
      }
    } else {
      // source = narrow: its dim g is the kept result dim of group g (or index 0 if none)
      tv->shape.assign(wide.shape.size(), Ref::value(1));
      for (size_t g = 0; g < groups.size(); ++g) {
        Index ix;
        if (keep[g] >= 0) {
          ix.dim = keep[g];
          tv->shape[(size_t)keep[g]] = src->shape[g];
        } else {
          ix.kind = Index::Const;
          ix.c = 0;
        }
        with[g] = ix;
      }
    }
    tv->expr = substitute(src->expr, with);
    defineTensor(result, tv);
  }

  Ref parseSliceEntry() {
    if (r_.peek() == '%') return extentOf(r_.ssa());
    return Ref::value(r_.integer());
  }
  std::vector<Ref> parseSliceList() {
    std::vector<Ref> v;
    r_.expect('[');
    if (!r_.eat(']')) {
      do v.push_back(parseSliceEntry()); while (r_.eat(','));
      r_.expect(']');
    }
    return v;
  }

  void parseExtractSlice(const std::string &result) {
    TensorP src = tensorOf(r_.ssa());
    std::vector<Ref> offsets = parseSliceList(), sizes = parseSliceList(), strides = parseSliceList();
    r_.expect(':');
    parseType();
    if (!r_.eatWord("to")) r_.fail("expected 'to' in tensor.extract_slice");
    TypeInfo rt = parseType();
    const size_t rank = src->shape.size();
    if (offsets.size() != rank || sizes.size() != rank || strides.size() != rank || rt.shape.size() != rank)
      r_.fail("tensor.extract_slice: rank-reducing or malformed slices are not supported");
    for (const Ref &s : strides)
      if (s.arg >= 0 || s.constant != 1) r_.fail("tensor.extract_slice: only unit strides are supported");
    if (!src->expr || src->reduced || !src->parts.empty()) r_.fail("tensor.extract_slice of this value is not supported");
    auto tv = std::make_shared<Tensor>();
    tv->elem = src->elem;
    tv->shape = sizes;
    tv->expr = offsetReads(src->expr, offsets);
    defineTensor(result, tv);
  }

  void parseConcat(const std::string &result) {
    if (!r_.eatWord("dim")) r_.fail("expected 'dim(N)' in tensor.concat");
    r_.expect('(');
    const int64_t dim = r_.integer();
    r_.expect(')');
    if (dim != 0) r_.fail("tensor.concat is supported along dim 0 only");
    auto tv = std::make_shared<Tensor>();
    do {
      TensorP p = tensorOf(r_.ssa());
      if (!p->expr || p->reduced || !p->parts.empty()) r_.fail("tensor.concat operand is not an elementwise value");
      tv->parts.push_back(p);
    } while (r_.eat(','));
    r_.expect(':');
    r_.expect('(');
    do parseType(); while (r_.eat(','));
    r_.expect(')');
    if (!r_.eatArrow()) r_.fail("expected '->' in tensor.concat");
    TypeInfo rt = parseType();
    tv->elem = rt.elemKnown ? rt.elem : tv->parts[0]->elem;
    tv->shape = tv->parts[0]->shape;
    defineTensor(result, tv);
  }

  // ---- linalg.generic ----
  void parseGeneric(const std::vector<std::string> &results) {
    std::vector<AffineMap> maps;
    std::vector<std::string> iterators;
    r_.expect('{');
    if (!r_.eat('}')) {
      for (;;) {
        std::string key = r_.ident();
        r_.expect('=');
        if (key == "indexing_maps") {
          r_.expect('[');
          do maps.push_back(parseMapRef()); while (r_.eat(','));
          r_.expect(']');
        } else if (key == "iterator_types") {
          r_.expect('[');
          do {
            if (r_.peek() == '"') {
              r_.eat('"');
              iterators.push_back(r_.ident());
              r_.expect('"');
            } else {
              r_.sigil('#', "an iterator type");   // #linalg.iterator_type<parallel>
              r_.expect('<');
              iterators.push_back(r_.ident());
              r_.expect('>');
            }
          } while (r_.eat(','));
          r_.expect(']');
        } else {
          r_.skipBalanced();
        }
        if (r_.eat('}')) break;
        r_.expect(',');
      }
    }
    Operands ins = parseOperandGroup("ins"), outs = parseOperandGroup("outs");
    if (r_.eatWord("attrs")) { r_.expect('='); r_.expect('{'); skipDict(); }
    if (outs.names.size() != 1 || results.size() != 1) r_.fail("linalg.generic with exactly one output is supported");
    if (maps.size() != ins.names.size() + 1) r_.fail("linalg.generic: one indexing map per operand is required");
    const int rank = (int)iterators.size();
    if (rank < 1 || rank > afir_region::kMaxRank) r_.fail("linalg.generic: iteration rank must be 1..3");
    for (AffineMap &m : maps) {
      // A map declared over more dims than there are iterators is taken as one over the
      // iterators when it uses no other dim: the reference's mean example reads its row sums
      // through the two-dim map (d0, d1) -> (d0) in a one-iterator generic
      // (examples/broadcast-add-reduce/step0_input_mean.mlir:76-80).
      bool inside = m.numDims > rank;
      for (const Index &ix : m.results) inside = inside && (ix.kind != Index::Dim || ix.dim < rank);
      if (inside) m.numDims = rank;
      if (m.numDims != rank) r_.fail("linalg.generic: affine map does not match the iterator count");
    }
    bool reduction = false;
    for (int i = 0; i < rank; ++i) {
      if (iterators[i] == "reduction") {
        if (i != rank - 1) r_.fail("only a reduction over the last iteration dim is supported");
        reduction = true;
      } else if (iterators[i] != "parallel") {
        r_.fail("unknown iterator type '" + iterators[i] + "'");
      }
    }
    std::vector<TensorP> inT;
    for (const std::string &n : ins.names) inT.push_back(tensorOf(n));
    TensorP outT = tensorOf(outs.names[0]);
    const AffineMap &outMap = maps.back();

    // region
    r_.expect('{');
    std::string bb = r_.sigil('^', "a block label");
    r_.expect('(');
    std::vector<std::string> blockArgs;
    if (!r_.eat(')')) {
      do {
        blockArgs.push_back(r_.ssa());
        r_.expect(':');
        parseType();
      } while (r_.eat(','));
      r_.expect(')');
    }
    r_.expect(':');
    if (blockArgs.size() != ins.names.size() + 1) r_.fail("linalg.generic: one block argument per operand is required");

    body_.clear();
    inBody_ = true;
    TensorP reducedOperand;   // set when an operand is the result of a reduction
    for (size_t i = 0; i < ins.names.size(); ++i) {
      Value v;
      const TensorP &t = inT[i];
      if ((int)maps[i].results.size() != (int)t->shape.size())
        r_.fail("linalg.generic: map of operand " + std::to_string(i) + " does not match its rank");
      if (!afir_region::isFloat(t->elem)) {
        // an index tensor: usable through arith.index_cast only
        if (t->directArg < 0 || t->shape.size() != 1 || maps[i].results[0].kind != Index::Dim)
          r_.fail("integer operands must be rank-1 function arguments read through a (d_k) map");
        v.kind = Value::IndexV;
        v.index.kind = Index::Gather;
        v.index.dim = maps[i].results[0].dim;
        v.index.indexArg = t->directArg;
        v.blockArgOperand = (int)i;
      } else {
        if (t->expr && t->reduced && t->parts.empty() && !reduction) {
          // the row sums of a reduction, consumed elementwise (mean = sum / N): the generic
          // must walk exactly the sums' index space and read nothing else
          if (reducedOperand || !maps[i].isIdentity() || rank != (int)t->shape.size())
            r_.fail("a reduced value can only be consumed through an identity map, once");
          reducedOperand = t;
          v.kind = Value::Scalar;
          auto e = std::make_shared<Expr>();
          e->kind = Expr::Reduced;
          // the sums sit in a tensor of t's element type before this generic reads them
          v.scalar = makeCast(t->elem, e);
          body_[blockArgs[i]] = v;
          continue;
        }
        if (!t->expr || t->reduced || !t->parts.empty())
          r_.fail("operand " + ins.names[i] + " is not an elementwise value (uninitialised, reduced or concatenated)");
        v.kind = Value::Scalar;
        v.scalar = substitute(t->expr, maps[i].results);
      }
      body_[blockArgs[i]] = v;
    }
    {
      Value acc;
      acc.kind = Value::Accumulator;
      body_[blockArgs.back()] = acc;
    }
    ExprP yielded;
    bool yieldedAccumulates = false;
    for (;;) {
      if (r_.peek() == '}') r_.fail("linalg.generic body has no linalg.yield");
      std::vector<std::string> res;
      if (r_.peek() == '%') {
        res.push_back(r_.ssa());
        r_.expect('=');
      }
      const std::string op = r_.ident();
      if (op == "linalg.yield") {
        Value &v = lookup(r_.ssa());
        r_.expect(':');
        parseType();
        if (v.kind == Value::Float) yielded = makeConst((float)v.number);
        else if (v.kind == Value::Scalar) yielded = v.scalar;
        else r_.fail("linalg.yield of a value that is not a scalar expression");
        yieldedAccumulates = v.blockArgOperand == -2;
        break;
      }
      if (res.size() != 1) r_.fail("operation '" + op + "' in a generic body must define one value");
      parseBodyOp(op, res[0], rank);
    }
    r_.expect('}');
    inBody_ = false;
    body_.clear();
    if (r_.eatArrow()) parseType();

    auto tv = std::make_shared<Tensor>();
    tv->elem = outT->elem;
    tv->shape = outT->shape;
    if (!reduction && reducedOperand) {
      if (yieldedAccumulates) r_.fail("a parallel generic must not read its output");
      if (!outMap.isIdentity()) r_.fail("linalg.generic: only an identity output map is supported for parallel generics");
      if (containsInput(yielded)) r_.fail("a generic that consumes a reduced value may combine it with constants and extents only");
      tv->reduced = true;
      tv->expr = reducedOperand->expr;
      tv->iterSizes = reducedOperand->iterSizes;
      // a tail on a tail: the earlier one takes the place of the sum
      tv->tail = reducedOperand->tail ? replaceReduced(yielded, reducedOperand->tail) : yielded;
    } else if (!reduction) {
      if (yieldedAccumulates) r_.fail("a parallel generic must not read its output");
      if (!outMap.isIdentity()) r_.fail("linalg.generic: only an identity output map is supported for parallel generics");
      tv->expr = yielded;
    } else {
      if (!yieldedAccumulates) r_.fail("a reduction generic must yield accumulator + value (arith.addf)");
      if ((int)outMap.results.size() != rank - 1) r_.fail("reduction output map must drop the reduced dim");
      for (int i = 0; i < rank - 1; ++i)
        if (outMap.results[i].kind != Index::Dim || outMap.results[i].dim != i)
          r_.fail("reduction output map must be (d0, ..., d_{n-2})");
      if (!(outT->filled && outT->fill == 0.f)) r_.fail("a reduction generic needs a zero-filled init (linalg.fill 0)");
      tv->reduced = true;
      tv->expr = yielded;
      tv->iterSizes = outT->shape;
      // extent of the reduced dim: from the first operand that is indexed by it
      Ref red;
      bool found = false;
      for (size_t i = 0; i < inT.size() && !found; ++i)
        for (size_t d = 0; d < maps[i].results.size() && !found; ++d)
          if (maps[i].results[d].kind == Index::Dim && maps[i].results[d].dim == rank - 1) {
            red = inT[i]->shape[d];
            found = true;
          }
      if (!found) r_.fail("no operand is indexed by the reduced dimension");
      tv->iterSizes.push_back(red);
    }
    defineTensor(results[0], tv);
  }

  OpCode binaryOp(const std::string &op) {
    static const struct { const char *n; OpCode c; } table[] = {
        {"arith.addf", OpCode::Add}, {"arith.subf", OpCode::Sub}, {"arith.mulf", OpCode::Mul},
        {"arith.divf", OpCode::Div}, {"arith.maximumf", OpCode::Max}, {"arith.minimumf", OpCode::Min}};
    for (const auto &e : table)
      if (op == e.n) return e.c;
    r_.fail("operation '" + op + "' has no HIP lowering inside a fused region");
  }

  void parseBodyOp(const std::string &op, const std::string &result, int rank) {
    Value out;
    if (op == "arith.constant") {
      parseConstant(result);
      return;
    }
    if (op == "linalg.index") {
      const int64_t k = r_.integer();
      r_.expect(':');
      parseType();
      if (k < 0 || k >= rank) r_.fail("linalg.index out of range");
      out.kind = Value::IndexV;
      out.index.kind = Index::Dim;
      out.index.dim = (int)k;
    } else if (op == "arith.index_cast") {
      Value &v = lookup(r_.ssa());
      r_.expect(':');
      parseType();
      if (!r_.eatWord("to")) r_.fail("expected 'to' in arith.index_cast");
      parseType();
      if (v.kind != Value::IndexV) r_.fail("arith.index_cast of a value that is not an index");
      out = v;
    } else if (op == "tensor.extract") {
      TensorP src = tensorOf(r_.ssa());
      r_.expect('[');
      std::vector<Index> idx;
      if (!r_.eat(']')) {
        do {
          Value &v = lookup(r_.ssa());
          if (v.kind == Value::IndexV) idx.push_back(v.index);
          else if (v.kind == Value::Int) { Index c; c.kind = Index::Const; c.c = (int64_t)v.number; idx.push_back(c); }
          else r_.fail("tensor.extract index must be linalg.index, a constant or a cast index-tensor element");
        } while (r_.eat(','));
        r_.expect(']');
      }
      r_.expect(':');
      parseType();
      if (!src->expr || src->reduced || !src->parts.empty() || idx.size() != src->shape.size())
        r_.fail("tensor.extract from this value is not supported");
      out.kind = Value::Scalar;
      out.scalar = substitute(src->expr, idx);
    } else if (op == "arith.negf") {
      Value &v = lookup(r_.ssa());
      r_.expect(':');
      parseType();
      out.kind = Value::Scalar;
      out.scalar = makeUnary(OpCode::Neg, scalarOf(v));
    } else if (op == "arith.truncf" || op == "arith.extf") {
      // mixed-precision chains: truncf rounds to the narrower type (nearest even); extf is
      // exact, the value is already one of the narrower type
      Value v = lookup(r_.ssa());
      r_.expect(':');
      parseType();
      if (!r_.eatWord("to")) r_.fail("expected 'to' in " + op);
      TypeInfo to = parseType();
      if (!to.elemKnown || !afir_region::isFloat(to.elem)) r_.fail(op + " to a type that is not f16, bf16 or f32");
      if (v.blockArgOperand == -2) r_.fail("the accumulated value may only be yielded");
      out.kind = Value::Scalar;
      out.scalar = op == "arith.truncf" ? makeCast(to.elem, scalarOf(v)) : scalarOf(v);
    } else {
      const OpCode code = binaryOp(op);
      Value a = lookup(r_.ssa());
      r_.expect(',');
      Value b = lookup(r_.ssa());
      if (r_.eatWord("fastmath")) r_.skipBalanced();
      r_.expect(':');
      parseType();
      out.kind = Value::Scalar;
      if (a.kind == Value::Accumulator || b.kind == Value::Accumulator) {
        if (code != OpCode::Add) r_.fail("only a sum reduction (arith.addf with the accumulator) is supported");
        const Value &other = a.kind == Value::Accumulator ? b : a;
        if (other.kind == Value::Accumulator) r_.fail("accumulator added to itself");
        out.scalar = scalarOf(other);
        out.blockArgOperand = -2;  // marks accumulator + value
      } else {
        if (a.blockArgOperand == -2 || b.blockArgOperand == -2)
          r_.fail("the accumulated value may only be yielded");
        out.scalar = makeBinary(code, scalarOf(a), scalarOf(b));
      }
    }
    body_[result] = out;
  }

  static bool containsInput(const ExprP &e) {
    if (e->kind == Expr::Input || e->kind == Expr::Matmul) return true;
    if (e->kind == Expr::Unary) return containsInput(e->a);
    if (e->kind == Expr::Binary) return containsInput(e->a) || containsInput(e->b);
    return false;
  }
  static bool containsReduced(const ExprP &e) {
    if (e->kind == Expr::Reduced) return true;
    if (e->kind == Expr::Unary) return containsReduced(e->a);
    if (e->kind == Expr::Binary) return containsReduced(e->a) || containsReduced(e->b);
    return false;
  }
  static ExprP replaceReduced(const ExprP &e, const ExprP &with) {
    if (e->kind == Expr::Reduced) return with;
    if (e->kind == Expr::Unary) return withOperand(e, replaceReduced(e->a, with));
    if (e->kind == Expr::Binary) {
      auto r = std::make_shared<Expr>(*e);
      r->a = replaceReduced(e->a, with);
      r->b = replaceReduced(e->b, with);
      return r;
    }
    return e;
  }

  ExprP scalarOf(const Value &v) {
    if (v.kind == Value::Scalar) return v.scalar;
    if (v.kind == Value::Float) return makeConst((float)v.number);
    if (v.kind == Value::ExtentFloat) {
      auto e = std::make_shared<Expr>();
      e->kind = Expr::ExtentConst;
      e->extent = v.extent;
      e->extentType = v.elem;
      return e;
    }
    r_.fail("expected a floating-point scalar");
  }

  // ---- AFIR ops (custom syntax) ----
  struct AfirAttrs {
    bool hasAxis = false;
    int64_t axis = 0;
    bool hasSlope = false;
    double slope = 0.0;
    bool hasConcatAxis = false;
    int64_t concatAxis = 0;
  };
  AfirAttrs parseAfirAttrs() {
    AfirAttrs a;
    if (!r_.eat('{')) return a;
    if (r_.eat('}')) return a;
    for (;;) {
      std::string key = r_.ident();
      r_.expect('=');
      if (key == "axis") {
        a.hasAxis = true;
        a.axis = r_.integer();
        if (r_.eat(':')) parseType();
      } else if (key == "concat_axis") {
        a.hasConcatAxis = true;
        a.concatAxis = r_.integer();
        if (r_.eat(':')) parseType();
      } else if (key == "negative_slop" || key == "negative_slope") {
        a.hasSlope = true;
        a.slope = r_.number();
        if (r_.eat(':')) parseType();
      } else {
        r_.skipBalanced();
      }
      if (r_.eat('}')) break;
      r_.expect(',');
    }
    return a;
  }

  // numpy-style broadcast of `t` to `rank` dims with result extents `shape`
  // (lib/Dialect/AFIR/Ops/Basic/math.cpp:274-381): trailing-aligned, a static
  // extent of 1 is read at index 0.
  ExprP broadcastTo(const TensorP &t, const std::vector<int64_t> &staticShape, int rank) {
    std::vector<Index> with;
    const int lead = rank - (int)t->shape.size();
    for (size_t d = 0; d < t->shape.size(); ++d) {
      Index ix;
      if (staticShape[d] == 1 && rank > 0) {
        ix.kind = Index::Const;
        ix.c = 0;
      } else {
        ix.dim = lead + (int)d;
      }
      with.push_back(ix);
    }
    return substitute(t->expr, with);
  }

  void parseAfir(const std::string &name, const std::string &result) {
    std::vector<std::string> operands;
    do operands.push_back(r_.ssa()); while (r_.eat(','));
    AfirAttrs attrs = parseAfirAttrs();
    r_.expect(':');
    if (name == "concat") {
      // afir.concat %a, %b, ... {concat_axis = 0 : i32} : ta, tb, ... -> tr: along the
      // rows it is the row-range segmentation of tensor.concat dim(0)
      if (!attrs.hasConcatAxis || attrs.concatAxis != 0) r_.fail("afir.concat is supported along axis 0 only");
      do parseType(); while (r_.eat(','));
      if (!r_.eatArrow()) r_.fail("expected '->' in afir.concat");
      TypeInfo rt = parseType();
      auto tv = std::make_shared<Tensor>();
      for (const std::string &o : operands) {
        TensorP p = tensorOf(o);
        if (!p->expr || p->reduced || !p->parts.empty()) r_.fail("afir.concat operand is not an elementwise value");
        tv->parts.push_back(p);
      }
      tv->elem = rt.elemKnown ? rt.elem : tv->parts[0]->elem;
      tv->shape = tv->parts[0]->shape;
      defineTensor(result, tv);
      return;
    }
    std::vector<TypeInfo> inTypes;
    if (r_.eat('(')) {
      do inTypes.push_back(parseType()); while (r_.eat(','));
      r_.expect(')');
    } else {
      inTypes.push_back(parseType());
    }
    if (!r_.eatArrow()) r_.fail("expected '->' in afir." + name);
    TypeInfo rt = parseType();
    if (inTypes.size() != operands.size()) r_.fail("afir." + name + ": operand / type count mismatch");
    std::vector<TensorP> in;
    for (const std::string &o : operands) {
      TensorP t = tensorOf(o);
      if (!t->expr || t->reduced || !t->parts.empty()) r_.fail("afir." + name + ": operand is not an elementwise value");
      if (inTypes[in.size()].shape.size() != t->shape.size())
        r_.fail("afir." + name + ": the type given for " + o + " has another rank than the value");
      in.push_back(t);
    }
    auto tv = std::make_shared<Tensor>();
    tv->elem = rt.elemKnown ? rt.elem : in[0]->elem;
    // integer tensors (include/Dialect/AFIR/Ops/Basic/math.td:71-98): add, sub, mul, maximum,
    // minimum, neg, relu, abs and the data movement ops; operands and result of one kind
    const bool integer = afir_region::isRegionInt(tv->elem);
    for (const TensorP &t : in)
      if (afir_region::isRegionInt(t->elem) != integer)
        r_.fail("afir." + name + ": integer and floating-point tensors in one operation");
    if (!integer && !afir_region::isFloat(tv->elem)) r_.fail("afir." + name + ": unsupported result element type");
    if (integer && (name == "div" || name == "truediv" || name == "leaky_relu" || name == "sum"))
      r_.fail("afir." + name + " on integer tensors has no HIP lowering");

    static const struct { const char *n; OpCode c; } binary[] = {
        {"add", OpCode::Add}, {"sub", OpCode::Sub}, {"mul", OpCode::Mul}, {"div", OpCode::Div},
        {"maximum", OpCode::Max}, {"minimum", OpCode::Min}, {"truediv", OpCode::Div}};
    for (const auto &b : binary) {
      if (name != b.n) continue;
      if (in.size() != 2) r_.fail("afir." + name + " takes two operands");
      const int rank = (int)std::max(in[0]->shape.size(), in[1]->shape.size());
      // result extents: per trailing-aligned dim, the operand whose extent is not a static 1
      tv->shape.assign(rank, Ref::value(1));
      for (int d = 0; d < rank; ++d) {
        for (int k = 0; k < 2; ++k) {
          const int own = d - (rank - (int)in[k]->shape.size());
          if (own < 0) continue;
          const int64_t st = inTypes[k].shape[own];
          if (st == 1) continue;
          tv->shape[d] = in[k]->shape[own];
          break;
        }
      }
      tv->expr = makeBinary(b.c, broadcastTo(in[0], inTypes[0].shape, rank),
                            broadcastTo(in[1], inTypes[1].shape, rank));
      defineTensor(result, tv);
      return;
    }
    {
      static const char *const unary[] = {"load", "store", "abs", "relu", "neg", "leaky_relu", "broadcast", "sum", "cast"};
      bool known = false;
      for (const char *u : unary) known = known || name == u;
      if (!known) r_.fail("afir." + name + " has no HIP lowering");
    }
    if (in.size() != 1) r_.fail("afir." + name + " takes one operand");
    if (name == "cast") {
      // include/Dialect/AFIR/Ops/Basic/cast.td:22-25, between the float types: the value
      // rounded to the result's element type (a widening cast changes nothing)
      if (integer || !afir_region::isFloat(in[0]->elem)) r_.fail("afir.cast between integer types has no HIP lowering");
      tv->shape = in[0]->shape;
      tv->expr = tv->elem == in[0]->elem ? in[0]->expr : makeCast(tv->elem, in[0]->expr);   // (to f32: exact, no cast)
    } else if (name == "load" || name == "store") {
      // data movement between global memory and the core in an AscGraph
      // (include/Dialect/AFIR/Ops/Basic/data.td:31-32): the value itself
      tv->shape = in[0]->shape;
      tv->expr = in[0]->expr;
    } else if (name == "abs") {
      // |x| = maximum(x, -x): exact, +0 for both zeros, NaN stays NaN
      tv->shape = in[0]->shape;
      tv->expr = makeBinary(OpCode::Max, in[0]->expr, makeUnary(OpCode::Neg, in[0]->expr));
    } else if (name == "relu" || name == "neg" || name == "leaky_relu") {
      tv->shape = in[0]->shape;
      if (name == "relu") tv->expr = makeUnary(OpCode::Relu, in[0]->expr);
      else if (name == "neg") tv->expr = makeUnary(OpCode::Neg, in[0]->expr);
      else {
        if (!attrs.hasSlope) r_.fail("afir.leaky_relu needs the negative_slop attribute");
        tv->expr = makeUnary(OpCode::Leaky, in[0]->expr, (float)attrs.slope);
      }
    } else if (name == "broadcast") {
      const int rank = (int)rt.shape.size();
      if (rank < (int)in[0]->shape.size()) r_.fail("afir.broadcast: result rank below input rank");
      const int lead = rank - (int)in[0]->shape.size();
      for (int d = 0; d < rank; ++d) {
        const int own = d - lead;
        if (rt.shape[d] >= 0 && !(own >= 0 && inTypes[0].shape[own] == rt.shape[d] && rt.shape[d] != 1))
          tv->shape.push_back(Ref::value(rt.shape[d]));
        else if (own >= 0 && inTypes[0].shape[own] != 1)
          tv->shape.push_back(in[0]->shape[own]);
        else if (rt.shape[d] >= 0)
          tv->shape.push_back(Ref::value(rt.shape[d]));
        else
          r_.fail("afir.broadcast: cannot tell the extent of a broadcast dim from a dynamic result type");
      }
      tv->expr = broadcastTo(in[0], inTypes[0].shape, rank);
    } else if (name == "sum") {
      const int rank = (int)in[0]->shape.size();
      if (!attrs.hasAxis) r_.fail("afir.sum needs the axis attribute");
      if (rank < 2 || attrs.axis != rank - 1) r_.fail("afir.sum is supported over the last axis of a rank >= 2 tensor");
      tv->reduced = true;
      tv->expr = in[0]->expr;
      tv->iterSizes = in[0]->shape;
      tv->shape.assign(in[0]->shape.begin(), in[0]->shape.end() - 1);
    } else {
      r_.fail("afir." + name + " has no HIP lowering");
    }
    defineTensor(result, tv);
  }

  // ---- emission ----
  static int stackNeed(const ExprP &e) {
    switch (e->kind) {
      case Expr::Unary: return stackNeed(e->a);
      case Expr::Binary: {
        const int a = stackNeed(e->a), b = stackNeed(e->b);
        const bool commutes = e->op == OpCode::Add || e->op == OpCode::Mul;
        if (commutes && b > a) return std::max(b, a + 1);
        return std::max(a, b + 1);
      }
      default: return 1;
    }
  }

  void emitExpr(const ExprP &e, std::vector<afir_region::Op> *ops) {
    afir_region::Op o;
    switch (e->kind) {
      case Expr::Constant:
        o.code = OpCode::Const;
        o.constant = e->value;
        ops->push_back(o);
        return;
      case Expr::Reduced:
        return;   // the row's sum: already on the stack when the tail starts
      case Expr::ExtentConst:
        o.code = OpCode::Const;
        o.extent = true;
        o.constRef = e->extent;
        o.constType = e->extentType;
        ops->push_back(o);
        return;
      case Expr::Matmul:
        if (!ops->empty()) r_.fail("a matmul must be the first value of its fused region");
        o.code = OpCode::Matmul;
        o.arg = e->arg;
        o.arg2 = e->arg2;
        o.transA = e->transA;
        o.transB = e->transB;
        ops->push_back(o);
        return;
      case Expr::Input: {
        o.code = OpCode::Push;
        o.arg = e->arg;
        for (const Index &ix : e->idx) {
          afir_region::MapResult m;
          if (ix.kind == Index::Dim) { m.kind = afir_region::MapResult::IterDim; m.iterDim = ix.dim; }
          else if (ix.kind == Index::Const) { m.kind = afir_region::MapResult::Constant; m.constant = ix.c; }
          else { m.kind = afir_region::MapResult::Gather; m.iterDim = ix.dim; m.indexArg = ix.indexArg; }
          o.map.push_back(m);
        }
        bool sliced = false;
        for (const Ref &s : e->slice) sliced |= s.arg >= 0 || s.constant != 0;
        if (sliced) o.slice = e->slice;
        ops->push_back(o);
        return;
      }
      case Expr::Unary:
        emitExpr(e->a, ops);
        o.code = e->op;
        o.constant = e->value;
        o.constType = e->extentType;   // Cast
        ops->push_back(o);
        return;
      case Expr::Binary: {
        // Evaluate the deeper operand first where the operation commutes
        // exactly (IEEE add and mul do), and a matmul before anything else.
        const bool commutes = e->op == OpCode::Add || e->op == OpCode::Mul;
        bool bFirst = false;
        if (commutes) {
          if (containsMatmul(e->b)) bFirst = true;
          else if (!containsMatmul(e->a) && stackNeed(e->b) > stackNeed(e->a)) bFirst = true;
        }
        // in a tail the sum is on the stack before anything else: it has to be the first
        // operand evaluated, which a commuting operation can arrange and 'c - sum' cannot
        if (containsReduced(e->b) && !containsReduced(e->a)) {
          if (e->op == OpCode::Sub) {   // c - s is (-s) + c, exactly
            emitExpr(e->b, ops);
            o.code = OpCode::Neg;
            ops->push_back(o);
            emitExpr(e->a, ops);
            o.code = OpCode::Add;
            ops->push_back(o);
            return;
          }
          if (e->op == OpCode::Div) r_.fail("a constant divided by a reduced value is not supported");
          bFirst = true;
        } else if (containsReduced(e->a)) {
          bFirst = false;
        }
        emitExpr(bFirst ? e->b : e->a, ops);
        emitExpr(bFirst ? e->a : e->b, ops);
        o.code = e->op;
        ops->push_back(o);
        return;
      }
    }
  }
  static bool containsMatmul(const ExprP &e) {
    if (e->kind == Expr::Matmul) return true;
    if (e->kind == Expr::Unary) return containsMatmul(e->a);
    if (e->kind == Expr::Binary) return containsMatmul(e->a) || containsMatmul(e->b);
    return false;
  }

  void emitSegment(const TensorP &t, const Ref &outOffset, afir_region::Program *p) {
    afir_region::Segment g;
    g.sizes = t->reduced ? t->iterSizes : t->shape;
    g.rank = (int)g.sizes.size();
    g.outOffset = outOffset;
    if (stackNeed(t->expr) > afir_region::kMaxStack)
      r_.fail("the fused expression needs more than " + std::to_string(afir_region::kMaxStack) + " live values");
    emitExpr(t->expr, &g.ops);
    afir_region::Op o;
    if (t->reduced) {
      o.code = OpCode::ReduceSum;
      g.ops.push_back(o);
      if (t->tail) emitExpr(t->tail, &g.ops);
    }
    // a last rounding to the output's own type is what the store does
    if (!g.ops.empty() && g.ops.back().code == OpCode::Cast && g.ops.back().constType == t->elem) g.ops.pop_back();
    o = afir_region::Op();
    o.code = OpCode::Store;
    g.ops.push_back(o);
    p->segments.push_back(std::move(g));
  }

  void emit(const TensorP &result, Translation *out) {
    afir_region::Program p;
    p.args = args_;
    afir_region::Arg o;
    o.isOutput = true;
    o.type = result->elem;
    o.rank = (int)result->shape.size();
    if (!afir_region::isFloat(o.type) && !afir_region::isRegionInt(o.type))
      r_.fail("the function must return an f16, bf16, f32, i16 or i32 tensor");
    p.args.push_back(o);
    if (!result->parts.empty()) {
      // first row of each part: the sum of the parts before it (constants folded)
      int64_t constant = 0;
      std::vector<Ref> terms;
      for (size_t i = 0; i < result->parts.size(); ++i) {
        const TensorP &part = result->parts[i];
        emitSegment(part, Ref::value(0), &p);
        afir_region::Segment &g = p.segments.back();
        if (terms.empty()) {
          g.outOffset = Ref::value(constant);
        } else {
          g.outOffset = terms[0];
          g.outOffsetMore.assign(terms.begin() + 1, terms.end());
          if (constant) g.outOffsetMore.push_back(Ref::value(constant));
        }
        const Ref &rows = part->shape[0];
        if (rows.arg < 0) constant += rows.constant;
        else terms.push_back(rows);
      }
    } else {
      if (!result->expr) r_.fail("the function returns an uninitialised tensor");
      emitSegment(result, Ref::value(0), &p);
    }
    std::string why = afir_region::validate(p);
    if (!why.empty()) r_.fail(why);
    out->program = std::move(p);
  }

  Reader r_;
  bool inModule_ = false;
  bool inBody_ = false;
  std::map<std::string, AffineMap> aliases_;
  std::map<std::string, Value> env_, body_;
  std::vector<afir_region::Arg> args_;
};

}  // namespace

std::string selectFunction(const std::string &text, const std::string &name) {
  // positions of `func.func` outside of comments
  std::vector<size_t> funcs;
  for (size_t at = text.find("func.func"); at != std::string::npos; at = text.find("func.func", at + 9)) {
    const size_t bol = text.rfind('\n', at);
    const size_t comment = text.find("//", bol == std::string::npos ? 0 : bol);
    if (comment == std::string::npos || comment > at) funcs.push_back(at);
  }
  if (funcs.empty()) return "";
  for (size_t at : funcs) {
    size_t p = at + 9;
    auto skipSpace = [&]() { while (p < text.size() && isspace((unsigned char)text[p])) ++p; };
    skipSpace();
    for (const char *vis : {"private", "public"})
      if (text.compare(p, std::strlen(vis), vis) == 0) { p += std::strlen(vis); skipSpace(); }
    if (p >= text.size() || text[p] != '@') continue;
    size_t e = p + 1;
    while (e < text.size() && (isalnum((unsigned char)text[e]) || text[e] == '_' || text[e] == '.' || text[e] == '$')) ++e;
    if (text.substr(p + 1, e - p - 1) == name) return text.substr(0, funcs[0]) + text.substr(at);
  }
  return "";
}

std::string translateMlirToRegion(const std::string &mlirText, Translation *out) {
  try {
    Translator t(mlirText);
    Translation tr;
    t.run(&tr);
    *out = std::move(tr);
    return "";
  } catch (const Failure &f) {
    return f.what();
  }
}

std::string tilingSpaceJson(const afir_region::Program &program, const std::string &kernelName) {
  std::string s = "{\n  \"kernel\": \"" + kernelName + "\",\n  \"soc\": \"gfx950\",\n  \"tiling_params\": [\n";
  const std::vector<std::string> names = afir_region::tilingFieldNames(program);
  for (size_t i = 0; i < names.size(); ++i)
    s += "    {\"name\": \"" + names[i] + "\", \"type\": \"int64\"}" + (i + 1 < names.size() ? ",\n" : "\n");
  s += "  ]\n}\n";
  return s;
}

}  // namespace afir_target
