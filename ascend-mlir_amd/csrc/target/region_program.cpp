// Fused-region programs: text form, validation and resolution against shapes
// (see region_program.h).  Host code only.
#include "region_program.h"

#include <algorithm>
#include <cerrno>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <sstream>

namespace afir_region {

const char *elemTypeName(ElemType t) {
  switch (t) {
    case ElemType::F16: return "f16";
    case ElemType::BF16: return "bf16";
    case ElemType::F32: return "f32";
    case ElemType::I32: return "i32";
    case ElemType::I64: return "i64";
    case ElemType::I16: return "i16";
  }
  return "f32";
}

size_t elemTypeBytes(ElemType t) {
  switch (t) {
    case ElemType::F16:
    case ElemType::BF16: return 2;
    case ElemType::F32:
    case ElemType::I32: return 4;
    case ElemType::I64: return 8;
    case ElemType::I16: return 2;
  }
  return 4;
}

bool parseElemType(const std::string &s, ElemType *out) {
  static const struct { const char *n; ElemType t; } table[] = {
      {"f16", ElemType::F16}, {"bf16", ElemType::BF16}, {"f32", ElemType::F32},
      {"i32", ElemType::I32}, {"i64", ElemType::I64}, {"i16", ElemType::I16}};
  for (const auto &e : table)
    if (s == e.n) { *out = e.t; return true; }
  return false;
}

bool Segment::reduces() const {
  for (const Op &o : ops)
    if (o.code == OpCode::ReduceSum) return true;
  return false;
}

namespace {

const struct { OpCode code; const char *name; } kSimpleOps[] = {
    {OpCode::Add, "add"}, {OpCode::Sub, "sub"}, {OpCode::Mul, "mul"}, {OpCode::Div, "div"},
    {OpCode::Max, "max"}, {OpCode::Min, "min"}, {OpCode::Relu, "relu"}, {OpCode::Neg, "neg"},
    {OpCode::Store, "store"}};

std::string refText(const Ref &r) {
  if (r.arg < 0) return std::to_string(r.constant);
  return "arg" + std::to_string(r.arg) + "." + std::to_string(r.dim);
}

bool parseInt(const std::string &s, int64_t *out) {
  if (s.empty()) return false;
  errno = 0;
  char *end = nullptr;
  long long v = std::strtoll(s.c_str(), &end, 10);
  if (errno || *end) return false;
  *out = v;
  return true;
}

bool parseRef(const std::string &s, Ref *out) {
  if (s.compare(0, 3, "arg") == 0) {
    size_t dot = s.find('.');
    if (dot == std::string::npos) return false;
    int64_t a, d;
    if (!parseInt(s.substr(3, dot - 3), &a) || !parseInt(s.substr(dot + 1), &d)) return false;
    if (a < 0 || d < 0) return false;
    *out = Ref::dimOf((int)a, (int)d);
    return true;
  }
  int64_t c;
  if (!parseInt(s, &c)) return false;
  *out = Ref::value(c);
  return true;
}

bool parseArgName(const std::string &s, int *out) {
  if (s.compare(0, 3, "arg") != 0) return false;
  int64_t a;
  if (!parseInt(s.substr(3), &a) || a < 0) return false;
  *out = (int)a;
  return true;
}

std::string floatText(float f) {
  char buf[48];
  std::snprintf(buf, sizeof buf, "%.9g", (double)f);
  return buf;
}

std::string err(int line, const std::string &msg) {
  return "region program line " + std::to_string(line) + ": " + msg;
}

}  // namespace

std::string serialize(const Program &p) {
  std::string s = "afir-hip-region 1\n";
  for (const Arg &a : p.args)
    s += std::string("arg ") + (a.isOutput ? "out " : "in ") + elemTypeName(a.type) + " " +
         std::to_string(a.rank) + "\n";
  for (const Segment &g : p.segments) {
    s += "segment " + std::to_string(g.rank) + "\n";
    s += "size";
    for (const Ref &r : g.sizes) s += " " + refText(r);
    s += "\noutoff " + refText(g.outOffset);
    for (const Ref &r : g.outOffsetMore) s += " " + refText(r);
    s += "\n";
    for (const Op &o : g.ops) {
      switch (o.code) {
        case OpCode::Push: {
          s += "push arg" + std::to_string(o.arg);
          for (const MapResult &m : o.map) {
            if (m.kind == MapResult::IterDim) s += " d" + std::to_string(m.iterDim);
            else if (m.kind == MapResult::Constant) s += " " + std::to_string(m.constant);
            else s += " g" + std::to_string(m.iterDim) + ":arg" + std::to_string(m.indexArg);
          }
          if (!o.slice.empty()) {
            s += " slice";
            for (const Ref &r : o.slice) s += " " + refText(r);
          }
          s += "\n";
          break;
        }
        case OpCode::Matmul:
          s += "matmul arg" + std::to_string(o.arg) + " arg" + std::to_string(o.arg2) +
               (o.transA ? " ta" : "") + (o.transB ? " tb" : "") + "\n";
          break;
        case OpCode::Const:
          if (o.extent)
            s += "const " + refText(o.constRef) +
                 (o.constType == ElemType::F32 ? std::string() : std::string(" ") + elemTypeName(o.constType)) + "\n";
          else
            s += "const " + floatText(o.constant) + "\n";
          break;
        case OpCode::Leaky: s += "leaky " + floatText(o.constant) + "\n"; break;
        case OpCode::Cast: s += std::string("cast ") + elemTypeName(o.constType) + "\n"; break;
        case OpCode::Dup: s += "dup " + std::to_string(o.depth) + "\n"; break;
        case OpCode::ReduceSum: s += "reduce sum\n"; break;
        default:
          for (const auto &e : kSimpleOps)
            if (e.code == o.code) s += std::string(e.name) + "\n";
      }
    }
    s += "end\n";
  }
  return s;
}

std::string parse(const std::string &text, Program *out) {
  Program p;
  std::istringstream in(text);
  std::string line;
  int lineno = 0;
  bool header = false;
  Segment *seg = nullptr;
  while (std::getline(in, line)) {
    ++lineno;
    size_t hash = line.find('#');
    if (hash != std::string::npos) line.erase(hash);
    std::istringstream ls(line);
    std::vector<std::string> tok;
    for (std::string t; ls >> t;) tok.push_back(t);
    if (tok.empty()) continue;
    if (!header) {
      if (tok.size() != 2 || tok[0] != "afir-hip-region" || tok[1] != "1")
        return err(lineno, "expected header 'afir-hip-region 1'");
      header = true;
      continue;
    }
    const std::string &k = tok[0];
    if (k == "arg") {
      if (seg || !p.segments.empty()) return err(lineno, "arg lines must precede the segments");
      Arg a;
      int64_t rank;
      if (tok.size() != 4 || (tok[1] != "in" && tok[1] != "out") || !parseElemType(tok[2], &a.type) ||
          !parseInt(tok[3], &rank))
        return err(lineno, "expected 'arg in|out <type> <rank>'");
      a.isOutput = tok[1] == "out";
      a.rank = (int)rank;
      p.args.push_back(a);
    } else if (k == "segment") {
      if (seg) return err(lineno, "segment inside a segment (missing 'end')");
      int64_t rank;
      if (tok.size() != 2 || !parseInt(tok[1], &rank)) return err(lineno, "expected 'segment <rank>'");
      p.segments.emplace_back();
      seg = &p.segments.back();
      seg->rank = (int)rank;
    } else if (!seg) {
      return err(lineno, "'" + k + "' outside a segment");
    } else if (k == "end") {
      seg = nullptr;
    } else if (k == "size") {
      seg->sizes.clear();
      for (size_t i = 1; i < tok.size(); ++i) {
        Ref r;
        if (!parseRef(tok[i], &r)) return err(lineno, "bad extent '" + tok[i] + "'");
        seg->sizes.push_back(r);
      }
    } else if (k == "outoff") {
      if (tok.size() < 2 || !parseRef(tok[1], &seg->outOffset)) return err(lineno, "expected 'outoff <ref> [<ref> ...]'");
      for (size_t i = 2; i < tok.size(); ++i) {
        Ref r;
        if (!parseRef(tok[i], &r)) return err(lineno, "bad output offset term '" + tok[i] + "'");
        seg->outOffsetMore.push_back(r);
      }
    } else if (k == "push") {
      Op o;
      o.code = OpCode::Push;
      if (tok.size() < 2 || !parseArgName(tok[1], &o.arg)) return err(lineno, "expected 'push arg<N> ...'");
      size_t i = 2;
      for (; i < tok.size() && tok[i] != "slice"; ++i) {
        MapResult m;
        const std::string &t = tok[i];
        int64_t v;
        if (t[0] == 'd' && parseInt(t.substr(1), &v)) {
          m.kind = MapResult::IterDim;
          m.iterDim = (int)v;
        } else if (t[0] == 'g') {
          size_t colon = t.find(':');
          if (colon == std::string::npos || !parseInt(t.substr(1, colon - 1), &v) ||
              !parseArgName(t.substr(colon + 1), &m.indexArg))
            return err(lineno, "bad gather map entry '" + t + "'");
          m.kind = MapResult::Gather;
          m.iterDim = (int)v;
        } else if (parseInt(t, &v)) {
          m.kind = MapResult::Constant;
          m.constant = v;
        } else {
          return err(lineno, "bad map entry '" + t + "'");
        }
        o.map.push_back(m);
      }
      if (i < tok.size()) {
        for (++i; i < tok.size(); ++i) {
          Ref r;
          if (!parseRef(tok[i], &r)) return err(lineno, "bad slice offset '" + tok[i] + "'");
          o.slice.push_back(r);
        }
      }
      seg->ops.push_back(o);
    } else if (k == "matmul") {
      Op o;
      o.code = OpCode::Matmul;
      if (tok.size() < 3 || tok.size() > 5 || !parseArgName(tok[1], &o.arg) || !parseArgName(tok[2], &o.arg2))
        return err(lineno, "expected 'matmul arg<A> arg<B> [ta] [tb]'");
      for (size_t i = 3; i < tok.size(); ++i) {
        if (tok[i] == "ta" && !o.transA && !o.transB) o.transA = true;
        else if (tok[i] == "tb" && !o.transB) o.transB = true;
        else return err(lineno, "expected 'matmul arg<A> arg<B> [ta] [tb]'");
      }
      seg->ops.push_back(o);
    } else if (k == "const" && tok.size() >= 2 && tok[1].compare(0, 3, "arg") == 0) {
      Op o;
      o.code = OpCode::Const;
      o.extent = true;
      if (tok.size() > 3 || !parseRef(tok[1], &o.constRef) || o.constRef.arg < 0)
        return err(lineno, "expected 'const arg<A>.<D> [f16|bf16|f32]'");
      if (tok.size() == 3 && (!parseElemType(tok[2], &o.constType) || !isFloat(o.constType)))
        return err(lineno, "an extent constant is rounded through f16, bf16 or f32");
      seg->ops.push_back(o);
    } else if (k == "const" || k == "leaky") {
      Op o;
      o.code = k == "const" ? OpCode::Const : OpCode::Leaky;
      if (tok.size() != 2) return err(lineno, "expected '" + k + " <float>'");
      char *end = nullptr;
      o.constant = std::strtof(tok[1].c_str(), &end);
      if (*end) return err(lineno, "bad number '" + tok[1] + "'");
      seg->ops.push_back(o);
    } else if (k == "cast") {
      Op o;
      o.code = OpCode::Cast;
      if (tok.size() != 2 || !parseElemType(tok[1], &o.constType) || !isFloat(o.constType))
        return err(lineno, "expected 'cast f16|bf16|f32'");
      seg->ops.push_back(o);
    } else if (k == "dup") {
      Op o;
      o.code = OpCode::Dup;
      int64_t d;
      if (tok.size() != 2 || !parseInt(tok[1], &d)) return err(lineno, "expected 'dup <n>'");
      o.depth = (int)d;
      seg->ops.push_back(o);
    } else if (k == "reduce") {
      if (tok.size() != 2 || tok[1] != "sum") return err(lineno, "only 'reduce sum' is supported");
      Op o;
      o.code = OpCode::ReduceSum;
      seg->ops.push_back(o);
    } else {
      bool found = false;
      for (const auto &e : kSimpleOps)
        if (k == e.name && tok.size() == 1) {
          Op o;
          o.code = e.code;
          seg->ops.push_back(o);
          found = true;
        }
      if (!found) return err(lineno, "unknown operation '" + line + "'");
    }
  }
  if (!header) return "region program: missing header 'afir-hip-region 1'";
  if (seg) return "region program: missing 'end' of the last segment";
  std::string v = validate(p);
  if (!v.empty()) return v;
  *out = std::move(p);
  return "";
}

std::string validate(const Program &p) {
  if (p.args.size() < 1) return "region program: no arguments";
  if ((int)p.args.size() > kMaxArgs) return "region program: too many arguments";
  for (size_t i = 0; i < p.args.size(); ++i) {
    const Arg &a = p.args[i];
    if (a.rank < 0 || a.rank > kMaxRank) return "region program: argument rank must be 0.." + std::to_string(kMaxRank);
    if (a.isOutput != (i + 1 == p.args.size()))
      return "region program: exactly one output, declared last, is supported";
  }
  const bool integer = isRegionInt(p.output().type);
  if (!isFloat(p.output().type) && !integer) return "region program: the output must be f16, bf16, f32, i16 or i32";
  if (p.segments.empty()) return "region program: no segment";
  auto refOk = [&](const Ref &r) {
    return r.arg < 0 ? r.constant >= 0
                     : (r.arg < (int)p.args.size() && r.dim >= 0 && r.dim < p.args[r.arg].rank);
  };
  for (const Segment &g : p.segments) {
    if (g.rank < 1 || g.rank > kMaxRank) return "region program: iteration rank must be 1.." + std::to_string(kMaxRank);
    if ((int)g.sizes.size() != g.rank) return "region program: 'size' needs one extent per iteration dim";
    for (const Ref &r : g.sizes)
      if (!refOk(r)) return "region program: bad extent reference";
    if (!refOk(g.outOffset)) return "region program: bad output offset reference";
    for (const Ref &r : g.outOffsetMore)
      if (!refOk(r)) return "region program: bad output offset reference";
    if (g.ops.empty() || g.ops.back().code != OpCode::Store) return "region program: a segment must end with 'store'";
    if ((int)g.ops.size() > kMaxOps) return "region program: too many operations in a segment";
    int depth = 0, pushes = 0, tailOps = 0, tailExtents = 0, extents = 0;
    bool reduced = false;
    // after 'reduce sum': which stack entries derive from the sum (exactly one does at any time)
    std::vector<bool> fromSum;
    for (size_t i = 0; i < g.ops.size(); ++i) {
      const Op &o = g.ops[i];
      if (reduced) {
        // the tail: the row's sum combined with constants and extents
        if (o.code == OpCode::Push || o.code == OpCode::Matmul || o.code == OpCode::ReduceSum)
          return "region program: after 'reduce sum' only operations on constants and extents may follow";
        // (operations among constants are folded when the shapes are known and do not count)
        switch (o.code) {
          case OpCode::Const:
            fromSum.push_back(false);
            if (o.extent && ++tailExtents > kMaxTailExtents)
              return "region program: more than " + std::to_string(kMaxTailExtents) + " extent constants after 'reduce sum'";
            break;
          case OpCode::Dup:
            if (o.depth >= 0 && o.depth < (int)fromSum.size()) {
              if (fromSum[fromSum.size() - 1 - o.depth])
                return "region program: the operations after 'reduce sum' must form a chain on the sum (no 'dup' of it)";
              fromSum.push_back(false);
            }
            break;
          case OpCode::Add: case OpCode::Sub: case OpCode::Mul: case OpCode::Div: case OpCode::Max: case OpCode::Min:
            if (fromSum.size() >= 2) {
              const bool b = fromSum.back();
              fromSum.pop_back();
              fromSum.back() = fromSum.back() || b;
              if (fromSum.back()) ++tailOps;
            }
            break;
          case OpCode::Relu: case OpCode::Leaky: case OpCode::Neg: case OpCode::Cast:
            if (!fromSum.empty() && fromSum.back()) ++tailOps;
            break;
          default: break;
        }
        if (tailOps > kMaxTailOps)
          return "region program: more than " + std::to_string(kMaxTailOps) + " operations on the sum after 'reduce sum'";
      }
      switch (o.code) {
        case OpCode::Push: {
          if (o.arg < 0 || o.arg >= p.numInputs()) return "region program: push of a non-input argument";
          const Arg &a = p.args[o.arg];
          if (integer ? !isRegionInt(a.type) : !isFloat(a.type))
            return integer ? "region program: an integer region reads i16 / i32 tensors only"
                           : "region program: pushed tensors must be f16, bf16 or f32";
          if ((int)o.map.size() != a.rank) return "region program: map needs one entry per dim of the input";
          if (!o.slice.empty() && (int)o.slice.size() != a.rank)
            return "region program: slice needs one offset per dim of the input";
          for (const Ref &r : o.slice)
            if (!refOk(r)) return "region program: bad slice reference";
          int gathers = 0;
          for (const MapResult &m : o.map) {
            if (m.kind == MapResult::Constant) {
              if (m.constant < 0) return "region program: negative constant index";
              continue;
            }
            if (m.iterDim < 0 || m.iterDim >= g.rank) return "region program: map refers to a missing iteration dim";
            if (m.kind == MapResult::Gather) {
              ++gathers;
              if (m.indexArg < 0 || m.indexArg >= p.numInputs()) return "region program: bad index tensor";
              const Arg &ia = p.args[m.indexArg];
              if (ia.rank != 1 || (ia.type != ElemType::I32 && ia.type != ElemType::I64))
                return "region program: an index tensor must be rank-1 i32 or i64";
            }
          }
          if (gathers > 1) return "region program: at most one gathered dim per read";
          ++depth;
          ++pushes;
          break;
        }
        case OpCode::Matmul: {
          if (integer) return "region program: 'matmul' is not available in an integer region";
          if (i != 0 || (g.rank != 2 && g.rank != 3))
            return "region program: 'matmul' must open a rank-2 segment (rank-3: batched)";
          for (int a : {o.arg, o.arg2}) {
            if (a < 0 || a >= p.numInputs()) return "region program: matmul of a non-input argument";
            if (p.args[a].rank != g.rank || !isFloat(p.args[a].type))
              return "region program: matmul operands must be float tensors of the segment's rank";
          }
          ++depth;
          break;
        }
        case OpCode::Const:
          if (o.extent) {
            if (integer) return "region program: an extent constant is not available in an integer region";
            if (!refOk(o.constRef) || o.constRef.arg < 0) return "region program: bad extent constant";
            if (++extents > kMaxSegmentExtents)
              return "region program: more than " + std::to_string(kMaxSegmentExtents) + " extent constants in a segment";
            ++depth;
            break;
          }
          if (integer && (o.constant != (float)(int32_t)o.constant || o.constant >= 2147483648.f || o.constant < -2147483648.f))
            return "region program: a constant of an integer region must be a 32-bit integer";
          ++depth;
          break;
        case OpCode::Dup:
          if (o.depth < 0 || o.depth >= depth) return "region program: dup beyond the stack";
          ++depth;
          break;
        case OpCode::Add: case OpCode::Sub: case OpCode::Mul: case OpCode::Div:
        case OpCode::Max: case OpCode::Min:
          if (integer && o.code == OpCode::Div) return "region program: 'div' is not available in an integer region";
          if (depth < 2) return "region program: binary operation on fewer than two values";
          --depth;
          break;
        case OpCode::Relu: case OpCode::Leaky: case OpCode::Neg: case OpCode::Cast:
          if (integer && o.code == OpCode::Leaky) return "region program: 'leaky' is not available in an integer region";
          if (integer && o.code == OpCode::Cast) return "region program: 'cast' is not available in an integer region";
          if (o.code == OpCode::Cast && !isFloat(o.constType)) return "region program: 'cast' to a type that is not f16, bf16 or f32";
          if (depth < 1) return "region program: unary operation on an empty stack";
          break;
        case OpCode::ReduceSum:
          if (integer) return "region program: 'reduce sum' is not available in an integer region";
          if (depth != 1) return "region program: 'reduce sum' needs exactly one value";
          if (g.rank < 2) return "region program: a reduction needs an iteration rank of at least 2";
          reduced = true;
          fromSum.assign(1, true);
          break;
        case OpCode::Store:
          if (i + 1 != g.ops.size()) return "region program: 'store' must be last";
          if (depth != 1) return "region program: 'store' needs exactly one value";
          break;
      }
      if (depth > kMaxStack) return "region program: expression needs more than " + std::to_string(kMaxStack) + " live values";
    }
    if (pushes > 8) return "region program: more than 8 reads in a segment";
    const int outRank = g.rank - (reduced ? 1 : 0);
    if (p.output().rank != outRank) return "region program: output rank does not match the segment";
  }
  return "";
}

float roundThroughType(float f, ElemType t) {
  if (t != ElemType::F16 && t != ElemType::BF16) return f;
  uint32_t x;
  std::memcpy(&x, &f, 4);
  if (t == ElemType::BF16) {
    if ((x & 0x7fffffffu) > 0x7f800000u) return f;   // nan
    x += 0x7fffu + ((x >> 16) & 1u);
    x &= 0xffff0000u;
    std::memcpy(&f, &x, 4);
    return f;
  }
  const uint32_t sign = x & 0x80000000u;
  x &= 0x7fffffffu;
  if (x >= 0x7f800000u) return f;                       // inf / nan
  if (x >= 0x477ff000u) {                               // rounds to >= 65520: inf
    const uint32_t inf = sign | 0x7f800000u;
    std::memcpy(&f, &inf, 4);
    return f;
  }
  if (x < 0x38800000u) {                                // f16 subnormal range: quantum 2^-24
    float a;
    std::memcpy(&a, &x, 4);
    const float q = std::nearbyintf(a * 16777216.0f) / 16777216.0f;
    return sign ? -q : q;
  }
  x += 0xfffu + ((x >> 13) & 1u);
  x &= ~0x1fffu;
  x |= sign;
  std::memcpy(&f, &x, 4);
  return f;
}

std::vector<std::string> tilingFieldNames(const Program &p) {
  std::vector<std::string> names;
  for (size_t a = 0; a < p.args.size(); ++a)
    for (int d = 0; d < p.args[a].rank; ++d)
      names.push_back("dim_arg" + std::to_string(a) + "_" + std::to_string(d));
  return names;
}

std::string resolve(const Program &p, const std::vector<int64_t> &dims, Resolved *out) {
  Resolved r;
  size_t at = 0;
  for (const Arg &a : p.args) {
    std::vector<int64_t> shape;
    unsigned __int128 n = 1;
    for (int d = 0; d < a.rank; ++d) {
      if (at >= dims.size()) return "region: tiling data holds too few dimensions";
      const int64_t v = dims[at++];
      if (v < 0 || v > ((int64_t)1 << 40)) return "region: extent out of range in tiling data";
      shape.push_back(v);
      n *= (unsigned __int128)v;
    }
    n *= elemTypeBytes(a.type);
    if (n > ((unsigned __int128)1 << 46)) return "region: tensor too large";
    r.shapes.push_back(shape);
    r.bytes.push_back((size_t)n);
  }
  if (at != dims.size()) return "region: tiling data holds too many dimensions";
  auto value = [&](const Ref &ref) { return ref.arg < 0 ? ref.constant : r.shapes[ref.arg][ref.dim]; };
  const std::vector<int64_t> &oshape = r.shapes.back();
  int64_t outRowElems = 1;
  for (size_t d = 1; d < oshape.size(); ++d) outRowElems *= oshape[d];

  std::vector<std::pair<int64_t, int64_t>> rowRanges;
  for (const Segment &g : p.segments) {
    ResolvedSegment s;
    s.rank = g.rank;
    s.reduce = g.reduces();
    s.outType = p.output().type;
    for (int k = 0; k < g.rank; ++k) s.size[k] = value(g.sizes[k]);
    const int outRank = g.rank - (s.reduce ? 1 : 0);
    int64_t off0 = value(g.outOffset);
    for (const Ref &r : g.outOffsetMore) off0 += value(r);
    if (outRank == 0) return "region: scalar outputs are not supported";
    for (int d = 1; d < outRank; ++d)
      if (oshape[d] != s.size[d]) return "region: segment extent does not match the output shape";
    if (off0 + s.size[0] > oshape[0]) return "region: segment writes beyond the output";
    rowRanges.push_back({off0, off0 + s.size[0]});
    s.outOffsetElems = off0 * outRowElems;
    s.outElems = s.size[0] * outRowElems;

    bool inTail = false;
    struct TailEntry { bool sum; float value; };
    std::vector<TailEntry> tailStack;
    for (const Op &o : g.ops) {
      ResolvedOp ro;
      ro.code = o.code;
      ro.constant = o.extent ? roundThroughType((float)value(o.constRef), o.constType) : o.constant;
      ro.depth = o.depth;
      ro.castType = o.constType;
      if (inTail && o.code != OpCode::Store) {
        // symbolic evaluation: entries are the running sum or float32 constants
        auto fold = [](OpCode c, float a, float b) {
          switch (c) {
            case OpCode::Add: return a + b;
            case OpCode::Sub: return a - b;
            case OpCode::Mul: return a * b;
            case OpCode::Div: return a / b;
            case OpCode::Max: return (a != a || b != b) ? a + b : (a == b ? (std::signbit(a) ? b : a) : (a > b ? a : b));
            default: return (a != a || b != b) ? a + b : (a == b ? (std::signbit(a) ? a : b) : (a < b ? a : b));
          }
        };
        switch (o.code) {
          case OpCode::Const: tailStack.push_back({false, ro.constant}); break;
          case OpCode::Dup: tailStack.push_back(tailStack[tailStack.size() - 1 - o.depth]); break;
          case OpCode::Relu: case OpCode::Leaky: case OpCode::Neg: case OpCode::Cast: {
            TailEntry &e = tailStack.back();
            if (e.sum) {
              s.tail.push_back({o.code, o.constant, false, o.constType});
            } else {
              const float v = e.value;
              e.value = o.code == OpCode::Cast ? roundThroughType(v, o.constType)
                        : o.code == OpCode::Neg ? -v : fold(OpCode::Max, v, o.code == OpCode::Relu ? 0.f : v * o.constant);
            }
            break;
          }
          default: {   // binary
            const TailEntry b = tailStack.back();
            tailStack.pop_back();
            TailEntry &a = tailStack.back();
            if (!a.sum && !b.sum) a.value = fold(o.code, a.value, b.value);
            else if (a.sum) s.tail.push_back({o.code, b.value, false});
            else {   // constant op sum
              s.tail.push_back({o.code, a.value, o.code == OpCode::Sub || o.code == OpCode::Div});
              a.sum = true;
            }
            break;
          }
        }
        continue;
      }
      if (o.code == OpCode::ReduceSum) {
        inTail = true;
        tailStack.assign(1, TailEntry{true, 0.f});
      }
      if (o.code == OpCode::Matmul) {
        const std::vector<int64_t> &sa = r.shapes[o.arg], &sb = r.shapes[o.arg2];
        const size_t b0 = sa.size() - 2;   // 1 with a leading batch dim
        const int64_t am = sa[b0 + (o.transA ? 1 : 0)], ak = sa[b0 + (o.transA ? 0 : 1)];
        const int64_t bk = sb[b0 + (o.transB ? 1 : 0)], bn = sb[b0 + (o.transB ? 0 : 1)];
        if (am != s.size[b0] || bn != s.size[b0 + 1] || ak != bk ||
            (b0 && (sa[0] != s.size[0] || sb[0] != s.size[0])))
          return "region: matmul operand shapes do not agree with the segment";
        ro.arg = o.arg;
        ro.arg2 = o.arg2;
        ro.k = ak;
        ro.batch = b0 ? s.size[0] : 1;
        ro.transA = o.transA;
        ro.transB = o.transB;
      }
      if (o.code == OpCode::Push) {
        const std::vector<int64_t> &shape = r.shapes[o.arg];
        ResolvedInput in;
        in.arg = o.arg;
        in.type = p.args[o.arg].type;
        int64_t stride = 1;
        for (int d = (int)shape.size() - 1; d >= 0; --d) {
          const MapResult &m = o.map[d];
          const int64_t start = o.slice.empty() ? 0 : value(o.slice[d]);
          if (m.kind == MapResult::IterDim) {
            if (s.size[m.iterDim] > 0 && start + s.size[m.iterDim] > shape[d])
              return "region: read of argument " + std::to_string(o.arg) + " runs past dim " + std::to_string(d);
            in.iterStride[m.iterDim] += stride;
            in.offset += start * stride;
          } else if (m.kind == MapResult::Constant) {
            if (m.constant + start >= shape[d] && s.outElems > 0)
              return "region: constant index of argument " + std::to_string(o.arg) + " is out of range";
            in.offset += (m.constant + start) * stride;
          } else {
            in.gatherIterDim = m.iterDim;
            in.gatherIndexArg = m.indexArg;
            in.gatherIndexType = p.args[m.indexArg].type;
            in.gatherStride = stride;
            if (start > shape[d]) return "region: slice of a gathered dim starts past its end";
            in.gatherExtent = shape[d] - start;  // valid indices are [0, extent)
            in.offset += start * stride;
            if (r.shapes[m.indexArg][0] < s.size[m.iterDim])
              return "region: index tensor is shorter than the iteration dim it indexes";
          }
          stride *= shape[d];
        }
        ro.input = (int)s.inputs.size();
        s.inputs.push_back(in);
      }
      s.ops.push_back(ro);
    }
    r.segments.push_back(std::move(s));
  }
  std::sort(rowRanges.begin(), rowRanges.end());
  int64_t next = 0;
  for (const auto &rr : rowRanges) {
    if (rr.first != next) return "region: segments do not tile the output rows exactly";
    next = rr.second;
  }
  if (next != oshape[0]) return "region: segments do not cover the output";
  *out = std::move(r);
  return "";
}

}  // namespace afir_region
