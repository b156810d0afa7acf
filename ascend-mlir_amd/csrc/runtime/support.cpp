// dtype helpers, npy container, JSON reader, tiling bytes, output comparator.
#include <cerrno>
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <sstream>

#include <sys/stat.h>
#include <unistd.h>

#include "runtime.h"

namespace afirt {

std::string format(const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  va_list ap2;
  va_copy(ap2, ap);
  int n = std::vsnprintf(nullptr, 0, fmt, ap);
  va_end(ap);
  std::string out(n > 0 ? (size_t)n : 0, '\0');
  if (n > 0) std::vsnprintf(out.data(), (size_t)n + 1, fmt, ap2);
  va_end(ap2);
  return out;
}

size_t dtypeBytes(DType d) {
  switch (d) {
    case DType::F16: return 2;
    case DType::BF16: return 2;
    case DType::F32: return 4;
    case DType::INT8: return 1;
    case DType::INT32: return 4;
    case DType::INT64: return 8;
  }
  return 0;
}

const char *dtypeName(DType d) {
  switch (d) {
    case DType::F16: return "f16";
    case DType::BF16: return "bf16";
    case DType::F32: return "f32";
    case DType::INT8: return "i8";
    case DType::INT32: return "i32";
    case DType::INT64: return "i64";
  }
  return "?";
}

Expected<DType> parseDType(const std::string &n) {
  if (n == "f16" || n == "float16" || n == "half") return DType::F16;
  if (n == "bf16" || n == "bfloat16") return DType::BF16;
  if (n == "f32" || n == "float32" || n == "float") return DType::F32;
  if (n == "i8" || n == "int8") return DType::INT8;
  if (n == "i32" || n == "int32") return DType::INT32;
  if (n == "i64" || n == "int64") return DType::INT64;
  return Status::error("unsupported dtype: " + n);
}

// ------------------------------------------------------------------- npy ----

namespace {

// value of  'key': ( ... )  /  'key': '...'  in a numpy header dict
bool headerTuple(const std::string &h, const std::string &key, std::string &out) {
  size_t p = h.find("'" + key + "'");
  if (p == std::string::npos) return false;
  p = h.find(':', p);
  if (p == std::string::npos) return false;
  size_t open = h.find_first_not_of(" \t", p + 1);
  if (open == std::string::npos || h[open] != '(') return false;
  size_t close = h.find(')', open);
  if (close == std::string::npos) return false;
  out = h.substr(open + 1, close - open - 1);
  return true;
}

bool headerQuoted(const std::string &h, const std::string &key, std::string &out) {
  size_t p = h.find("'" + key + "'");
  if (p == std::string::npos) return false;
  p = h.find(':', p);
  if (p == std::string::npos) return false;
  size_t open = h.find_first_not_of(" \t", p + 1);
  if (open == std::string::npos || h[open] != '\'') return false;
  size_t close = h.find('\'', open + 1);
  if (close == std::string::npos || close == open + 1) return false;
  out = h.substr(open + 1, close - open - 1);
  return true;
}

}  // namespace

Expected<NDArray> LoadNpy(const std::string &path) {
  std::ifstream f(path, std::ios::binary);
  if (!f) return Status::error("Cannot open: " + path);
  char magic[6] = {0};
  f.read(magic, 6);
  if (f.gcount() != 6 || std::memcmp(magic, "\x93NUMPY", 6) != 0)
    return Status::error("Not a .npy file: " + path);
  uint8_t major = 0, minor = 0;
  f.read(reinterpret_cast<char *>(&major), 1);
  f.read(reinterpret_cast<char *>(&minor), 1);
  uint32_t hlen = 0;
  if (major == 1) {
    uint16_t h16 = 0;
    f.read(reinterpret_cast<char *>(&h16), 2);
    hlen = h16;
  } else {
    f.read(reinterpret_cast<char *>(&hlen), 4);
  }
  if (!f) return Status::error("Truncated header in: " + path);
  std::string header(hlen, '\0');
  f.read(header.data(), hlen);
  if (f.gcount() != (std::streamsize)hlen) return Status::error("Truncated header in: " + path);

  NDArray arr;
  std::string shapeText;
  if (!headerTuple(header, "shape", shapeText)) return Status::error("Cannot parse shape: " + path);
  {
    std::istringstream ss(shapeText);
    std::string tok;
    while (std::getline(ss, tok, ',')) {
      size_t b = tok.find_first_not_of(" \t");
      if (b == std::string::npos) continue;
      size_t e = tok.find_last_not_of(" \t");
      tok = tok.substr(b, e - b + 1);
      char *end = nullptr;
      errno = 0;
      long long v = std::strtoll(tok.c_str(), &end, 10);
      if (errno || end == tok.c_str() || *end != '\0' || v < 0)
        return Status::error("Cannot parse shape: " + path);
      arr.shape.push_back(v);
    }
  }
  std::string descr;
  if (!headerQuoted(header, "descr", descr)) return Status::error("Cannot parse dtype: " + path);
  if (descr == "<f2" || descr == "=f2") arr.dtype = DType::F16;
  else if (descr == "<V2" || descr == "=V2" || descr == "|V2") arr.dtype = DType::BF16;  // numpy has no bf16
  else if (descr == "<f4" || descr == "=f4") arr.dtype = DType::F32;
  else if (descr == "<i1" || descr == "=i1" || descr == "|i1") arr.dtype = DType::INT8;
  else if (descr == "<i4" || descr == "=i4") arr.dtype = DType::INT32;
  else if (descr == "<i8" || descr == "=i8") arr.dtype = DType::INT64;
  else return Status::error("Unsupported dtype '" + descr + "': " + path);
  if (header.find("'fortran_order': True") != std::string::npos)
    return Status::error("Fortran-order arrays are not supported: " + path);

  arr.allocate();
  f.read(reinterpret_cast<char *>(arr.data), (std::streamsize)arr.nbytes());
  if (f.gcount() != (std::streamsize)arr.nbytes()) return Status::error("Truncated data in: " + path);
  return arr;
}

Status SaveNpy(const std::string &path, const NDArray &arr) {
  const char *descr = nullptr;
  switch (arr.dtype) {
    case DType::F16: descr = "<f2"; break;
    case DType::BF16: descr = "<V2"; break;
    case DType::F32: descr = "<f4"; break;
    case DType::INT8: descr = "|i1"; break;
    case DType::INT32: descr = "<i4"; break;
    case DType::INT64: descr = "<i8"; break;
  }
  std::string shape = "(";
  for (size_t i = 0; i < arr.shape.size(); ++i) {
    shape += std::to_string(arr.shape[i]);
    if (arr.shape.size() == 1 || i + 1 < arr.shape.size()) shape += ",";
  }
  shape += ")";
  std::string dict = std::string("{'descr': '") + descr + "', 'fortran_order': False, 'shape': " +
                     shape + ", }";
  // 10-byte prefix + header is padded to a multiple of 64, newline-terminated
  size_t total = 10 + dict.size() + 1;
  dict.append((64 - total % 64) % 64, ' ');
  dict += '\n';
  if (dict.size() > 0xffff) return Status::error("npy header too large: " + path);

  // write next to the target and rename over it, so readers never see a torn file
  std::string tmp = path + "." + std::to_string((long)getpid()) + ".tmp";
  {
    std::ofstream f(tmp, std::ios::binary | std::ios::trunc);
    if (!f) return Status::error("Cannot write: " + tmp);
    uint16_t hlen = (uint16_t)dict.size();
    f.write("\x93NUMPY", 6);
    f.put(1);
    f.put(0);
    f.write(reinterpret_cast<const char *>(&hlen), 2);
    f.write(dict.data(), (std::streamsize)dict.size());
    if (arr.nbytes()) f.write(reinterpret_cast<const char *>(arr.data), (std::streamsize)arr.nbytes());
    f.close();
    if (!f) {
      std::remove(tmp.c_str());
      return Status::error("Cannot finalize temp npy file: " + tmp);
    }
  }
  if (std::rename(tmp.c_str(), path.c_str()) != 0) {
    std::remove(tmp.c_str());
    return Status::error("Cannot replace npy output: " + path);
  }
  return Status::success();
}

// ------------------------------------------------------------------ json ----

namespace {

struct JsonParser {
  const std::string &s;
  size_t i = 0;
  std::string err;

  void ws() {
    while (i < s.size() && (s[i] == ' ' || s[i] == '\t' || s[i] == '\n' || s[i] == '\r')) ++i;
  }
  bool fail(const std::string &m) {
    if (err.empty()) err = m + " at offset " + std::to_string(i);
    return false;
  }
  bool parseString(std::string &out) {
    if (i >= s.size() || s[i] != '"') return fail("expected string");
    ++i;
    while (i < s.size() && s[i] != '"') {
      char c = s[i++];
      if (c == '\\') {
        if (i >= s.size()) return fail("bad escape");
        char e = s[i++];
        switch (e) {
          case '"': out += '"'; break;
          case '\\': out += '\\'; break;
          case '/': out += '/'; break;
          case 'b': out += '\b'; break;
          case 'f': out += '\f'; break;
          case 'n': out += '\n'; break;
          case 'r': out += '\r'; break;
          case 't': out += '\t'; break;
          case 'u': {
            if (i + 4 > s.size()) return fail("bad \\u escape");
            unsigned cp = (unsigned)std::strtoul(s.substr(i, 4).c_str(), nullptr, 16);
            i += 4;
            if (cp < 0x80) out += (char)cp;
            else if (cp < 0x800) { out += (char)(0xC0 | (cp >> 6)); out += (char)(0x80 | (cp & 0x3F)); }
            else { out += (char)(0xE0 | (cp >> 12)); out += (char)(0x80 | ((cp >> 6) & 0x3F)); out += (char)(0x80 | (cp & 0x3F)); }
            break;
          }
          default: return fail("bad escape");
        }
      } else {
        out += c;
      }
    }
    if (i >= s.size()) return fail("unterminated string");
    ++i;
    return true;
  }
  bool parseValue(Json &v, int depth) {
    if (depth > 64) return fail("nesting too deep");
    ws();
    if (i >= s.size()) return fail("unexpected end");
    char c = s[i];
    if (c == '{') {
      v.kind = Json::Object;
      ++i;
      ws();
      if (i < s.size() && s[i] == '}') { ++i; return true; }
      while (true) {
        ws();
        std::string key;
        if (!parseString(key)) return false;
        ws();
        if (i >= s.size() || s[i] != ':') return fail("expected ':'");
        ++i;
        Json child;
        if (!parseValue(child, depth + 1)) return false;
        v.object.emplace_back(std::move(key), std::move(child));
        ws();
        if (i < s.size() && s[i] == ',') { ++i; continue; }
        if (i < s.size() && s[i] == '}') { ++i; return true; }
        return fail("expected ',' or '}'");
      }
    }
    if (c == '[') {
      v.kind = Json::Array;
      ++i;
      ws();
      if (i < s.size() && s[i] == ']') { ++i; return true; }
      while (true) {
        Json child;
        if (!parseValue(child, depth + 1)) return false;
        v.array.push_back(std::move(child));
        ws();
        if (i < s.size() && s[i] == ',') { ++i; continue; }
        if (i < s.size() && s[i] == ']') { ++i; return true; }
        return fail("expected ',' or ']'");
      }
    }
    if (c == '"') {
      v.kind = Json::String;
      return parseString(v.string);
    }
    if (s.compare(i, 4, "true") == 0) { v.kind = Json::Bool; v.boolean = true; i += 4; return true; }
    if (s.compare(i, 5, "false") == 0) { v.kind = Json::Bool; v.boolean = false; i += 5; return true; }
    if (s.compare(i, 4, "null") == 0) { v.kind = Json::Null; i += 4; return true; }
    if (c == '-' || (c >= '0' && c <= '9')) {
      size_t b = i;
      if (s[i] == '-') ++i;
      bool integral = true;
      while (i < s.size() && ((s[i] >= '0' && s[i] <= '9') || s[i] == '.' || s[i] == 'e' ||
                              s[i] == 'E' || s[i] == '+' || s[i] == '-')) {
        if (s[i] == '.' || s[i] == 'e' || s[i] == 'E') integral = false;
        ++i;
      }
      std::string tok = s.substr(b, i - b);
      char *end = nullptr;
      v.kind = Json::Number;
      v.number = std::strtod(tok.c_str(), &end);
      if (end == tok.c_str() || *end != '\0') return fail("bad number");
      if (integral) {
        errno = 0;
        long long iv = std::strtoll(tok.c_str(), &end, 10);
        if (!errno && *end == '\0') { v.is_integer = true; v.integer = iv; }
      }
      return true;
    }
    return fail("unexpected character");
  }
};

}  // namespace

Expected<Json> parseJson(const std::string &text) {
  JsonParser p{text};
  Json root;
  if (!p.parseValue(root, 0)) return Status::error("JSON parse error: " + p.err);
  p.ws();
  if (p.i != text.size()) return Status::error("JSON parse error: trailing characters at offset " + std::to_string(p.i));
  return root;
}

const Json *Json::get(const std::string &key) const {
  if (kind != Object) return nullptr;
  for (const auto &kv : object)
    if (kv.first == key) return &kv.second;
  return nullptr;
}
std::optional<std::string> Json::getString(const std::string &key) const {
  const Json *v = get(key);
  if (!v || v->kind != String) return std::nullopt;
  return v->string;
}
std::optional<int64_t> Json::getInteger(const std::string &key) const {
  const Json *v = get(key);
  if (!v || v->kind != Number) return std::nullopt;
  if (v->is_integer) return v->integer;
  if (std::floor(v->number) == v->number) return (int64_t)v->number;
  return std::nullopt;
}
std::optional<double> Json::getNumber(const std::string &key) const {
  const Json *v = get(key);
  if (!v || v->kind != Number) return std::nullopt;
  return v->number;
}
std::optional<bool> Json::getBoolean(const std::string &key) const {
  const Json *v = get(key);
  if (!v || v->kind != Bool) return std::nullopt;
  return v->boolean;
}
const Json *Json::getArray(const std::string &key) const {
  const Json *v = get(key);
  return (v && v->kind == Array) ? v : nullptr;
}
const Json *Json::getObject(const std::string &key) const {
  const Json *v = get(key);
  return (v && v->kind == Object) ? v : nullptr;
}

Expected<std::string> readTextFile(const std::string &path) {
  std::ifstream f(path, std::ios::binary);
  if (!f) return Status::error("cannot open '" + path + "'");
  std::ostringstream ss;
  ss << f.rdbuf();
  return ss.str();
}

// ---------------------------------------------------------------- tiling ----

Expected<TilingSchema> TilingSchema::fromJson(const std::string &path) {
  auto text = readTextFile(path);
  if (!text) return Status::error(text.error());
  auto parsed = parseJson(*text);
  if (!parsed) return Status::error("JSON parse error in '" + path + "': " + parsed.error());
  if (parsed->kind != Json::Object) return Status::error("'" + path + "': root must be a JSON object");
  const Json *params = parsed->getArray("tiling_params");
  if (!params) return Status::error("'" + path + "': missing 'tiling_params' array");
  TilingSchema schema;
  for (const Json &e : params->array) {
    if (e.kind != Json::Object)
      return Status::error("'" + path + "': tiling_params entry is not an object");
    auto name = e.getString("name");
    if (!name) return Status::error("'" + path + "': tiling_params entry missing 'name'");
    TilingField f;
    f.name = *name;
    if (auto type = e.getString("type")) f.type = *type;
    schema.fields_.push_back(std::move(f));
  }
  return schema;
}

TilingSchema TilingSchema::fromFields(std::vector<TilingField> fields) {
  TilingSchema s;
  s.fields_ = std::move(fields);
  return s;
}

Expected<std::vector<uint8_t>> TilingSchema::pack(
    const std::vector<std::pair<std::string, int64_t>> &params) const {
  if (params.size() != fields_.size()) {
    std::string msg = "tiling param count mismatch: got " + std::to_string(params.size()) +
                      ", expected " + std::to_string(fields_.size()) + " (";
    for (size_t i = 0; i < fields_.size(); ++i) {
      if (i) msg += ", ";
      msg += fields_[i].name;
    }
    msg += ")";
    return Status::error(msg);
  }
  std::vector<uint8_t> bytes;
  for (size_t i = 0; i < fields_.size(); ++i) {
    if (params[i].first != fields_[i].name)
      return Status::error("tiling param name mismatch at position " + std::to_string(i) +
                           ": got '" + params[i].first + "', expected '" + fields_[i].name + "'");
    const int64_t val = params[i].second;
    if (fields_[i].type == "int32" || fields_[i].type == "int32_t") {
      int32_t v = (int32_t)val;
      uint8_t buf[4];
      std::memcpy(buf, &v, 4);
      bytes.insert(bytes.end(), buf, buf + 4);
    } else {
      uint8_t buf[8];
      std::memcpy(buf, &val, 8);
      bytes.insert(bytes.end(), buf, buf + 8);
    }
  }
  return bytes;
}

Expected<std::vector<uint8_t>> packTilingBytes(const std::optional<TilingBinding> &tiling) {
  if (!tiling) return std::vector<uint8_t>{};
  if (!tiling->binaryPath.empty()) {
    std::ifstream f(tiling->binaryPath, std::ios::binary);
    if (!f) return Status::error("cannot read tiling binary: " + tiling->binaryPath);
    std::vector<uint8_t> bytes((std::istreambuf_iterator<char>(f)), std::istreambuf_iterator<char>());
    return bytes;
  }
  if (!tiling->schemaPath.empty()) {
    auto schema = TilingSchema::fromJson(tiling->schemaPath);
    if (!schema) return Status::error(schema.error());
    std::map<std::string, int64_t> parsed;
    std::istringstream ss(tiling->params);
    std::string tok;
    while (std::getline(ss, tok, ',')) {
      if (tok.empty()) continue;
      size_t eq = tok.find('=');
      if (eq == std::string::npos) return Status::error("tiling params token missing '=': " + tok);
      char *end = nullptr;
      errno = 0;
      long long v = std::strtoll(tok.c_str() + eq + 1, &end, 10);
      if (errno || end == tok.c_str() + eq + 1 || *end != '\0')
        return Status::error("tiling params value is not an integer: " + tok);
      parsed[tok.substr(0, eq)] = v;
    }
    std::vector<std::pair<std::string, int64_t>> ordered;
    for (const auto &field : schema->fields()) {
      auto it = parsed.find(field.name);
      if (it == parsed.end()) return Status::error("tiling params missing field: " + field.name);
      ordered.emplace_back(it->first, it->second);
    }
    return schema->pack(ordered);
  }
  if (!tiling->params.empty())
    return Status::error("tiling params require either a schema path or a binary path");
  return std::vector<uint8_t>{};
}

// ------------------------------------------------------------ comparator ----

namespace {

float widen(const void *base, size_t idx, DType dtype) {
  const uint8_t *p = static_cast<const uint8_t *>(base);
  switch (dtype) {
    case DType::F16: {
      uint16_t h;
      std::memcpy(&h, p + idx * 2, 2);
      uint32_t sign = (h >> 15) & 1, exp = (h >> 10) & 0x1f, frac = h & 0x3ff, f;
      if (exp == 0) f = (sign << 31) | (frac << 13);  // as the reference decodes it
      else if (exp == 31) f = (sign << 31) | 0x7f800000u | (frac << 13);
      else f = (sign << 31) | ((exp + 112) << 23) | (frac << 13);
      float r;
      std::memcpy(&r, &f, 4);
      return r;
    }
    case DType::BF16: {
      uint16_t h;
      std::memcpy(&h, p + idx * 2, 2);
      uint32_t f = (uint32_t)h << 16;
      float r;
      std::memcpy(&r, &f, 4);
      return r;
    }
    case DType::F32: { float v; std::memcpy(&v, p + idx * 4, 4); return v; }
    case DType::INT8: { int8_t v; std::memcpy(&v, p + idx, 1); return (float)v; }
    case DType::INT32: { int32_t v; std::memcpy(&v, p + idx * 4, 4); return (float)v; }
    case DType::INT64: { int64_t v; std::memcpy(&v, p + idx * 8, 8); return (float)v; }
  }
  return 0.f;
}

}  // namespace

Expected<OutputComparisonResult> compareRuntimeOutputs(const std::vector<NDArray> &actual,
                                                       const std::vector<NDArray> &expected,
                                                       double atol, double rtol) {
  if (actual.size() != expected.size())
    return Status::error(format("output count mismatch: got %zu, expected %zu", actual.size(),
                                expected.size()));
  OutputComparisonResult result;
  result.passed = true;
  double total = 0.0;
  size_t count = 0;
  for (size_t k = 0; k < actual.size(); ++k) {
    const NDArray &a = actual[k], &e = expected[k];
    if (a.shape != e.shape) return Status::error(format("output %zu shape mismatch", k));
    if (a.dtype != e.dtype) return Status::error(format("output %zu dtype mismatch", k));
    if (a.nbytes() != e.nbytes()) return Status::error(format("output %zu byte-size mismatch", k));
    const size_t n = a.numElements();
    if (n && (!a.data || !e.data)) return Status::error(format("output %zu has null data pointer", k));
    count += n;
    for (size_t i = 0; i < n; ++i) {
      const double av = (double)widen(a.data, i, a.dtype);
      const double ev = (double)widen(e.data, i, e.dtype);
      const double diff = std::abs(av - ev);
      total += diff;
      result.maxAbsDiff = std::max(result.maxAbsDiff, diff);
      if (diff > atol + rtol * std::abs(ev)) {
        result.passed = false;
        ++result.mismatches;
      }
    }
  }
  result.meanAbsDiff = count == 0 ? 0.0 : total / (double)count;
  if (!result.passed)
    result.errorMessage = format("output comparison failed: max_abs_diff=%g, mean_abs_diff=%g",
                                 result.maxAbsDiff, result.meanAbsDiff);
  return result;
}

}  // namespace afirt
