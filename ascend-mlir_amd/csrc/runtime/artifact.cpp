// Artifact directories and run manifests.
//
// On this backend the fused kernels are precompiled in the kernel library, so
// "compiling" a fused region means recognising which kernel family it is and
// writing an artifact that names it:
//     <root>/<kernel_name>.hipk      descriptor (key=value text)
//     <root>/out/manifest.txt        kernel_name= soc_version= kernel_kind=
//                                    device_binary_path= manifest_path=
//                                    kernel_so_path= kernel_so_symbol=
// The first five manifest keys are the reference's
// (lib/Runtime/Artifact/VecCubeArtifactBackend.cpp:62-106); kernel_so_path is
// the key its mix artifacts use for a launcher library
// (lib/Runtime/Artifact/RuntimeSessionRequestBuilder.cpp:374-455).
#include <dlfcn.h>
#include <sys/stat.h>

#include <cstring>
#include <fstream>
#include <sstream>

#include "runtime.h"

namespace afirt {

const char *kernelKindName(KernelKind k) {
  switch (k) {
    case KernelKind::Vec: return "vec";
    case KernelKind::Cube: return "cube";
    case KernelKind::Mix: return "mix";
  }
  return "vec";
}

Expected<KernelKind> parseKernelKind(const std::string &name) {
  if (name == "vec") return KernelKind::Vec;
  if (name == "cube") return KernelKind::Cube;
  if (name == "mix") return KernelKind::Mix;
  return Status::error("unsupported kernel kind: " + name);
}

namespace {

struct KnownKernel {
  const char *name;
  const char *symbol;
  KernelKind kind;
};
// Mirrors the registry of the kernel library (afir_hip_kernel_info); kept here
// so that artifacts can be written on a machine without the library loaded.
const KnownKernel kKnown[] = {
    {"fused_add_mul", "afir_hip_launch_fused_add_mul", KernelKind::Vec},
    {"broadcast_add_reducesum", "afir_hip_launch_broadcast_add_reducesum", KernelKind::Vec},
    {"relu_broadcast_add_transpose", "afir_hip_launch_relu_broadcast_add_transpose", KernelKind::Vec},
    {"gather_scale_shift", "afir_hip_launch_gather_scale_shift", KernelKind::Vec},
    {"matmul_add_leakyrelu", "afir_hip_launch_matmul_add_leakyrelu", KernelKind::Mix},
};

const KnownKernel *findKnown(const std::string &name) {
  for (const auto &k : kKnown)
    if (name == k.name) return &k;
  return nullptr;
}

bool makeDirs(const std::string &path) {
  std::string cur;
  for (size_t i = 0; i <= path.size(); ++i) {
    if (i == path.size() || path[i] == '/') {
      if (!cur.empty() && cur != "/") {
        if (mkdir(cur.c_str(), 0777) != 0 && errno != EEXIST) return false;
      }
    }
    if (i < path.size()) cur += path[i];
  }
  struct stat st;
  return stat(path.c_str(), &st) == 0 && S_ISDIR(st.st_mode);
}

std::string trim(const std::string &s) {
  size_t b = s.find_first_not_of(" \t\r\n");
  if (b == std::string::npos) return "";
  size_t e = s.find_last_not_of(" \t\r\n");
  return s.substr(b, e - b + 1);
}

std::map<std::string, std::string> parseKeyValues(const std::string &text) {
  std::map<std::string, std::string> kv;
  std::istringstream ss(text);
  std::string line;
  while (std::getline(ss, line)) {
    line = trim(line);
    if (line.empty() || line[0] == '#') continue;
    size_t eq = line.find('=');
    if (eq == std::string::npos) continue;
    kv[trim(line.substr(0, eq))] = trim(line.substr(eq + 1));
  }
  return kv;
}

std::string joinPath(const std::string &a, const std::string &b) {
  if (a.empty()) return b;
  if (!b.empty() && b[0] == '/') return b;
  return a.back() == '/' ? a + b : a + "/" + b;
}

bool fileExists(const std::string &p) {
  struct stat st;
  return stat(p.c_str(), &st) == 0 && S_ISREG(st.st_mode);
}

// first `func.func @name` in MLIR text
std::string firstFuncName(const std::string &text) {
  size_t p = text.find("func.func");
  while (p != std::string::npos) {
    size_t at = text.find('@', p);
    if (at == std::string::npos) return "";
    size_t e = at + 1;
    while (e < text.size() && (isalnum((unsigned char)text[e]) || text[e] == '_' || text[e] == '.' ||
                               text[e] == '$'))
      ++e;
    if (e > at + 1) return text.substr(at + 1, e - at - 1);
    p = text.find("func.func", e);
  }
  return "";
}

// argument names of the first func.func, in order: (%a: ..., %b: ...) -> {"%a", "%b"}
std::vector<std::string> firstFuncArgs(const std::string &text) {
  std::vector<std::string> args;
  size_t p = text.find("func.func");
  if (p == std::string::npos) return args;
  size_t open = text.find('(', p);
  if (open == std::string::npos) return args;
  int depth = 0;
  size_t i = open;
  std::string cur;
  for (; i < text.size(); ++i) {
    char c = text[i];
    if (c == '(' || c == '<' || c == '[' || c == '{') {
      if (depth++ > 0) cur += c;
    } else if (c == ')' || c == '>' || c == ']' || c == '}') {
      if (--depth == 0) break;
      cur += c;
    } else if (c == ',' && depth == 1) {
      args.push_back(cur);
      cur.clear();
    } else {
      cur += c;
    }
  }
  if (!trim(cur).empty()) args.push_back(cur);
  for (auto &a : args) {
    size_t c = a.find("//");
    while (c != std::string::npos) {  // drop trailing comments inside the signature
      size_t nl = a.find('\n', c);
      a.erase(c, nl == std::string::npos ? std::string::npos : nl - c);
      c = a.find("//");
    }
    size_t colon = a.find(':');
    a = trim(colon == std::string::npos ? a : a.substr(0, colon));
  }
  return args;
}

// %r = afir.<op> %x, %y ...   ->   (result, op, lhs, rhs)
struct AfirBinary {
  std::string result, op, lhs, rhs;
};
std::vector<AfirBinary> afirBinaries(const std::string &text) {
  std::vector<AfirBinary> ops;
  std::istringstream ss(text);
  std::string line;
  while (std::getline(ss, line)) {
    size_t c = line.find("//");
    if (c != std::string::npos) line = line.substr(0, c);
    size_t p = line.find("afir.");
    size_t eq = line.find('=');
    if (p == std::string::npos || eq == std::string::npos || eq > p) continue;
    AfirBinary b;
    b.result = trim(line.substr(0, eq));
    size_t e = p + 5;
    while (e < line.size() && (isalnum((unsigned char)line[e]) || line[e] == '_')) ++e;
    b.op = line.substr(p + 5, e - p - 5);
    std::string rest = line.substr(e);
    size_t stop = rest.find_first_of("{:");
    if (stop != std::string::npos) rest = rest.substr(0, stop);
    size_t comma = rest.find(',');
    if (comma == std::string::npos) continue;
    b.lhs = trim(rest.substr(0, comma));
    b.rhs = trim(rest.substr(comma + 1));
    if (!b.result.empty() && b.result[0] == '%' && !b.lhs.empty() && !b.rhs.empty()) ops.push_back(b);
  }
  return ops;
}

}  // namespace

std::string defaultKernelLibraryPath() {
  if (const char *env = std::getenv("AFIR_HIP_KERNELS_LIB"))
    if (*env) return env;
  Dl_info info;
  if (dladdr(reinterpret_cast<const void *>(&defaultKernelLibraryPath), &info) && info.dli_fname) {
    std::string self = info.dli_fname;
    size_t slash = self.rfind('/');
    if (slash != std::string::npos) {
      std::string candidate = self.substr(0, slash + 1) + "libafir_hip_kernels.so";
      if (fileExists(candidate)) return candidate;
    }
  }
  return "libafir_hip_kernels.so";
}

std::string serializeDescriptor(const HipKernelDescriptor &d) {
  std::string s = "afir-hip-artifact 1\n";
  s += "kernel_name=" + d.kernelName + "\n";
  s += "hip_kernel=" + d.hipKernel + "\n";
  s += "library=" + d.library + "\n";
  s += "symbol=" + d.symbol + "\n";
  return s;
}

Expected<HipKernelDescriptor> parseDescriptor(const std::string &text) {
  if (text.compare(0, 17, "afir-hip-artifact") != 0)
    return Status::error("not an afir-hip artifact descriptor (missing 'afir-hip-artifact' header)");
  auto kv = parseKeyValues(text.substr(text.find('\n') == std::string::npos ? text.size()
                                                                           : text.find('\n') + 1));
  HipKernelDescriptor d;
  d.kernelName = kv["kernel_name"];
  d.hipKernel = kv["hip_kernel"];
  d.library = kv["library"];
  d.symbol = kv["symbol"];
  if (d.hipKernel.empty()) return Status::error("artifact descriptor names no hip_kernel");
  const KnownKernel *k = findKnown(d.hipKernel);
  if (!k) return Status::error("artifact descriptor names an unknown hip_kernel: " + d.hipKernel);
  if (d.symbol.empty()) d.symbol = k->symbol;
  if (d.kernelName.empty()) d.kernelName = d.hipKernel;
  return d;
}

Expected<std::string> selectHipKernel(const std::string &text, const std::string &nameHint) {
  // 1. an explicit request
  for (const auto &kv : parseKeyValues(text))
    if (kv.first == "hip_kernel") {
      if (!findKnown(kv.second)) return Status::error("unknown hip_kernel: " + kv.second);
      return kv.second;
    }
  // 2. the AFIR elementwise chain %1 = afir.mul(afir.add(%a, %b), %b)
  //    (README.md:191-197 of the reference)
  auto ops = afirBinaries(text);
  if (ops.size() == 2 && ops[0].op == "add" && ops[1].op == "mul") {
    // The kernel computes (in0 + in1) * in1 with inputs bound in function
    // argument order, so the factor the product repeats must be the second
    // argument (the sum itself commutes bit-exactly).
    const auto &add = ops[0], &mul = ops[1];
    const auto args = firstFuncArgs(text);
    const std::string factor = mul.lhs == add.result ? mul.rhs : (mul.rhs == add.result ? mul.lhs : "");
    const bool sum_of_args = args.size() == 2 && ((add.lhs == args[0] && add.rhs == args[1]) ||
                                                  (add.lhs == args[1] && add.rhs == args[0]));
    if (sum_of_args && factor == args[1]) return std::string("fused_add_mul");
    return Status::error("afir add->mul chain is not of the form (arg0 + arg1) * arg1");
  }
  if (!ops.empty())
    return Status::error("unsupported AFIR elementwise chain (" + std::to_string(ops.size()) +
                         " ops); only afir.add -> afir.mul as (a + b) * b is lowered");
  // 3. a function named after a kernel family
  std::string fn = firstFuncName(text);
  if (!fn.empty() && findKnown(fn)) return fn;
  if (!nameHint.empty() && findKnown(nameHint)) return nameHint;
  return Status::error("cannot map kernel source to a fused HIP kernel (function '" + fn +
                       "'); known kernels: fused_add_mul, broadcast_add_reducesum, "
                       "relu_broadcast_add_transpose, gather_scale_shift, matmul_add_leakyrelu");
}

Expected<KernelArtifact> compileArtifact(const CompileRequest &request) {
  if (request.kernelSource.empty()) return Status::error("kernel source is required");
  if (request.outputDir.empty()) return Status::error("output directory is required");
  auto text = readTextFile(request.kernelSource);
  if (!text) return Status::error("cannot read kernel source: " + request.kernelSource);
  auto family = selectHipKernel(*text, request.kernelName);
  if (!family) return Status::error(family.error());
  const KnownKernel *known = findKnown(*family);

  std::string name = request.kernelName;
  if (name.empty()) name = firstFuncName(*text);
  if (name.empty()) name = *family;

  if (!makeDirs(joinPath(request.outputDir, "out")))
    return Status::error("cannot create artifact manifest directory");

  HipKernelDescriptor d;
  d.kernelName = name;
  d.hipKernel = *family;
  d.library = defaultKernelLibraryPath();
  d.symbol = known->symbol;
  const std::string binRel = name + ".hipk";
  const std::string binPath = joinPath(request.outputDir, binRel);
  {
    std::ofstream f(binPath, std::ios::binary | std::ios::trunc);
    if (!f) return Status::error("cannot write artifact descriptor: " + binPath);
    f << serializeDescriptor(d);
  }
  KernelArtifact a;
  a.kernelName = name;
  a.kernelKind = request.kernelKind ? *request.kernelKind : known->kind;
  a.socVersion = request.socVersion.empty() ? "gfx950" : request.socVersion;
  a.artifactRoot = request.outputDir;
  a.deviceBinaryPath = binPath;
  a.sharedLibraryPath = d.library;
  a.sharedLibrarySymbol = d.symbol;
  a.manifestPath = joinPath(request.outputDir, "out/manifest.txt");
  {
    std::ofstream f(a.manifestPath, std::ios::trunc);
    if (!f) return Status::error("cannot write artifact manifest");
    f << "kernel_name=" << a.kernelName << "\n";
    f << "soc_version=" << a.socVersion << "\n";
    f << "kernel_kind=" << kernelKindName(a.kernelKind) << "\n";
    f << "device_binary_path=" << binRel << "\n";
    f << "manifest_path=out/manifest.txt\n";
    f << "kernel_so_path=" << a.sharedLibraryPath << "\n";
    f << "kernel_so_symbol=" << a.sharedLibrarySymbol << "\n";
  }
  return a;
}

Expected<KernelArtifact> loadArtifactFromRoot(const std::string &root) {
  if (root.empty()) return Status::error("artifact root is required");
  const std::string manifestPath = joinPath(root, "out/manifest.txt");
  auto text = readTextFile(manifestPath);
  if (!text) return Status::error("cannot read artifact manifest: " + manifestPath);
  auto kv = parseKeyValues(*text);
  KernelArtifact a;
  a.artifactRoot = root;
  a.manifestPath = manifestPath;
  a.kernelName = kv["kernel_name"];
  if (a.kernelName.empty()) return Status::error("artifact manifest missing kernel_name: " + manifestPath);
  a.socVersion = kv.count("soc_version") ? kv["soc_version"] : "gfx950";
  if (kv.count("kernel_kind")) {
    auto kind = parseKernelKind(kv["kernel_kind"]);
    if (!kind) return Status::error(kind.error());
    a.kernelKind = *kind;
  }
  if (kv["device_binary_path"].empty())
    return Status::error("artifact manifest missing device_binary_path: " + manifestPath);
  a.deviceBinaryPath = joinPath(root, kv["device_binary_path"]);
  if (!fileExists(a.deviceBinaryPath))
    return Status::error("artifact device binary does not exist: " + a.deviceBinaryPath);
  a.sharedLibraryPath = kv["kernel_so_path"];
  a.sharedLibrarySymbol = kv["kernel_so_symbol"];
  auto dtext = readTextFile(a.deviceBinaryPath);
  if (!dtext) return Status::error(dtext.error());
  auto d = parseDescriptor(*dtext);
  if (!d) return Status::error(d.error() + ": " + a.deviceBinaryPath);
  if (a.sharedLibraryPath.empty()) a.sharedLibraryPath = d->library;
  if (a.sharedLibraryPath.empty()) a.sharedLibraryPath = defaultKernelLibraryPath();
  if (a.sharedLibrarySymbol.empty()) a.sharedLibrarySymbol = d->symbol;
  return a;
}

// ---------------------------------------------------------- run manifest ----

namespace {

Expected<std::vector<TensorBinding>> parseBindings(const Json &root, const char *field) {
  std::vector<TensorBinding> out;
  const Json *arr = root.getArray(field);
  if (!arr) return out;
  for (const Json &v : arr->array) {
    if (v.kind != Json::Object) return Status::error(std::string(field) + " entries must be objects");
    TensorBinding b;
    auto name = v.getString("name");
    if (!name) return Status::error("missing required string field: name");
    b.name = *name;
    std::string source = v.getString("source").value_or("external_file");
    if (source == "external_file") {
      if (auto p = v.getString("path")) b.path = *p;
    } else if (source == "task_output") {
      return Status::error("tensor binding source 'task_output' needs a multi-task session, which "
                           "this runtime does not run");
    } else {
      return Status::error("unsupported tensor binding source: " + source);
    }
    if (const Json *shape = v.getArray("shape")) {
      for (const Json &d : shape->array) {
        if (d.kind != Json::Number || !d.is_integer || d.integer < 0)
          return Status::error("shape entries must be non-negative integers");
        b.shape.push_back(d.integer);
      }
    }
    if (auto dt = v.getString("dtype")) {
      auto parsed = parseDType(*dt);
      if (!parsed) return Status::error(parsed.error());
      b.dtype = *parsed;
    }
    out.push_back(std::move(b));
  }
  return out;
}

Expected<RunTaskSpec> parseTask(const Json &root, const std::optional<std::string> &defaultRoot) {
  RunTaskSpec spec;
  auto id = root.getString("task_id");
  if (!id) return Status::error("missing required string field: task_id");
  spec.taskId = *id;
  if (auto r = root.getString("artifact_root")) spec.artifactRoot = *r;
  else if (defaultRoot) spec.artifactRoot = *defaultRoot;
  else return Status::error("missing required string field: artifact_root");
  if (const Json *deps = root.getArray("dependencies"))
    for (const Json &d : deps->array) {
      if (d.kind != Json::String) return Status::error("dependencies entries must be strings");
      spec.dependencies.push_back(d.string);
    }
  auto in = parseBindings(root, "inputs");
  if (!in) return Status::error(in.error());
  spec.invocation.inputs = std::move(*in);
  auto out = parseBindings(root, "outputs");
  if (!out) return Status::error(out.error());
  spec.invocation.outputs = std::move(*out);
  auto exp = parseBindings(root, "expected_outputs");
  if (!exp) return Status::error(exp.error());
  spec.invocation.expectedOutputs = std::move(*exp);
  if (const Json *t = root.get("tiling")) {
    if (t->kind != Json::Object) return Status::error("tiling must be an object");
    TilingBinding tb;
    tb.schemaPath = t->getString("schema").value_or("");
    tb.params = t->getString("params").value_or("");
    tb.binaryPath = t->getString("binary").value_or("");
    spec.invocation.tiling = tb;
  }
  if (auto v = root.getInteger("block_dim")) spec.invocation.blockDim = (int)*v;
  if (auto v = root.getInteger("workspace_size")) {
    if (*v < 0) return Status::error("workspace_size must be non-negative");
    spec.invocation.workspaceSize = (size_t)*v;
  }
  if (auto v = root.getBoolean("profiling")) spec.invocation.enableProfiling = *v;
  if (auto v = root.getNumber("atol")) spec.invocation.atol = *v;
  if (auto v = root.getNumber("rtol")) spec.invocation.rtol = *v;
  return spec;
}

}  // namespace

Expected<RunManifestSpec> loadRunManifest(const std::string &path) {
  auto text = readTextFile(path);
  if (!text) return Status::error("cannot read run manifest: " + path);
  auto json = parseJson(*text);
  if (!json) return Status::error("invalid JSON in run manifest: " + path);
  if (json->kind != Json::Object) return Status::error("run manifest root must be an object: " + path);
  RunManifestSpec spec;
  auto backend = json->getString("backend");
  if (!backend) return Status::error("missing required string field: backend");
  if (*backend != "hip" && *backend != "sim" && *backend != "npu")
    return Status::error("unsupported backend: " + *backend);
  spec.backend = *backend;
  std::optional<std::string> defaultRoot = json->getString("artifact_root");
  if (const Json *tasks = json->getArray("tasks")) {
    for (const Json &t : tasks->array) {
      if (t.kind != Json::Object) return Status::error("tasks entries must be objects");
      auto task = parseTask(t, defaultRoot);
      if (!task) return Status::error(task.error());
      spec.tasks.push_back(std::move(*task));
    }
  } else {
    auto task = parseTask(*json, defaultRoot);
    if (!task) return Status::error(task.error());
    spec.tasks.push_back(std::move(*task));
  }
  if (spec.tasks.empty()) return Status::error("run manifest must contain at least one task");
  return spec;
}

}  // namespace afirt
