// Artifact directories and run manifests.
//
// "Compiling" a fused region means translating its IR to a region program
// (csrc/target/mlir_translate.h) -- or taking an explicit request for one of
// the hand-tuned kernel families of the kernel library -- emitting HIP source
// specialised for the program (csrc/target/hip_emitter.h), compiling that with
// hipcc and writing an artifact that carries it all:
//     <root>/<kernel_name>.hipk      descriptor (key=value text, then the
//                                    region program after a "program:" line)
//     <root>/<kernel_name>.hip       emitted kernel source    } region programs,
//     <root>/<kernel_name>.hsaco     its gfx950 code object   } when hipcc is there
//     <root>/out/manifest.txt        kernel_name= soc_version= kernel_kind=
//                                    device_binary_path= manifest_path=
//                                    kernel_so_path= kernel_so_symbol=
// The first five manifest keys are the reference's
// (lib/Runtime/Artifact/VecCubeArtifactBackend.cpp:62-106); kernel_so_path is
// the key its mix artifacts use for a launcher library
// (lib/Runtime/Artifact/RuntimeSessionRequestBuilder.cpp:374-455).
#include <dlfcn.h>
#include <fcntl.h>
#include <spawn.h>
#include <sys/stat.h>
#include <sys/wait.h>
#include <unistd.h>

#include <cerrno>
#include <climits>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <sstream>

#include "../target/hip_emitter.h"
#include "../target/hiprtc_compile.h"
#include "../target/mlir_translate.h"

extern char **environ;
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
    {"fused_region", "afir_hip_launch_region", KernelKind::Vec},
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
  if (!d.codeObject.empty()) {
    s += "code_object=" + d.codeObject + "\n";
    s += "code_object_dir=" + d.codeObjectDir + "\n";
    if (d.codeObjectPreferred) s += "code_object_preferred=1\n";
  }
  if (!d.program.empty()) s += "program:\n" + d.program;
  return s;
}

Expected<HipKernelDescriptor> parseDescriptor(const std::string &text) {
  if (text.compare(0, 17, "afir-hip-artifact") != 0)
    return Status::error("not an afir-hip artifact descriptor (missing 'afir-hip-artifact' header)");
  std::string head = text, program;
  const size_t mark = text.find("\nprogram:\n");
  if (mark != std::string::npos) {
    head = text.substr(0, mark + 1);
    program = text.substr(mark + 10);
  }
  auto kv = parseKeyValues(head.substr(head.find('\n') == std::string::npos ? head.size()
                                                                           : head.find('\n') + 1));
  HipKernelDescriptor d;
  d.kernelName = kv["kernel_name"];
  d.hipKernel = kv["hip_kernel"];
  d.library = kv["library"];
  d.symbol = kv["symbol"];
  d.program = program;
  d.codeObject = kv["code_object"];
  d.codeObjectDir = kv["code_object_dir"];
  d.codeObjectPreferred = kv["code_object_preferred"] == "1";
  if (d.hipKernel.empty()) return Status::error("artifact descriptor names no hip_kernel");
  const KnownKernel *k = findKnown(d.hipKernel);
  if (!k) return Status::error("artifact descriptor names an unknown hip_kernel: " + d.hipKernel);
  if ((d.hipKernel == "fused_region") != !d.program.empty())
    return Status::error("artifact descriptor: a region program is required for fused_region and only there");
  if (d.symbol.empty()) d.symbol = k->symbol;
  if (d.kernelName.empty()) d.kernelName = d.hipKernel;
  return d;
}

namespace {
std::string absolutePath(const std::string &path) {
  char buf[PATH_MAX];
  return realpath(path.c_str(), buf) ? std::string(buf) : path;
}
}  // namespace

std::string resolveCodeObject(const HipKernelDescriptor &d, const std::string &descriptorDir) {
  if (d.codeObject.empty()) return "";
  if (!descriptorDir.empty() && fileExists(joinPath(descriptorDir, d.codeObject)))
    return joinPath(descriptorDir, d.codeObject);
  if (!d.codeObjectDir.empty() && fileExists(joinPath(d.codeObjectDir, d.codeObject)))
    return joinPath(d.codeObjectDir, d.codeObject);
  return "";
}

Expected<std::string> compileRegionCodeObject(const std::string &programText, const std::string &dir,
                                              const std::string &name,
                                              const std::map<std::string, int64_t> &emitOptions) {
  if (const char *env = std::getenv("AFIR_HIP_CODEGEN"))
    if (*env == '0') return Status::error("disabled by AFIR_HIP_CODEGEN=0");
  afir_region::Program program;
  if (std::string why = afir_region::parse(programText, &program); !why.empty()) return Status::error(why);
  afir_target::EmitOptions options;
  for (const auto &kv : emitOptions)
    if (!afir_target::setEmitOption(&options, kv.first, kv.second))
      return Status::error("unknown emit option '" + kv.first + "' (tile_p, tile_q, unroll)");
  std::string source;
  if (std::string why = afir_target::emitHipSource(program, name, &source, options); !why.empty())
    return Status::error(why);
  const std::string srcPath = joinPath(dir, name + ".hip"), objName = name + ".hsaco",
                    objPath = joinPath(dir, objName), logPath = joinPath(dir, name + ".hipcc.log");
  {
    std::ofstream f(srcPath, std::ios::trunc);
    if (!f) return Status::error("cannot write " + srcPath);
    f << source;
  }
  std::string hipcc;
  if (const char *env = std::getenv("HIPCC")) hipcc = env;
  if (hipcc.empty()) {
    const char *path = std::getenv("PATH");
    std::istringstream dirs(path ? path : "");
    for (std::string d; std::getline(dirs, d, ':');)
      if (!d.empty() && access(joinPath(d, "hipcc").c_str(), X_OK) == 0) {
        hipcc = joinPath(d, "hipcc");
        break;
      }
  }
  if (hipcc.empty() && access("/opt/rocm/bin/hipcc", X_OK) == 0) hipcc = "/opt/rocm/bin/hipcc";
  // No hipcc on this host (or AFIR_HIP_COMPILER=hiprtc): the runtime-compilation library of the
  // HIP runtime compiles the same source with the same options inside the process.
  const char *which = std::getenv("AFIR_HIP_COMPILER");
  const bool wantRtc = which && std::string(which) == "hiprtc", onlyHipcc = which && std::string(which) == "hipcc";
  if (onlyHipcc && hipcc.empty()) return Status::error("hipcc not found (set HIPCC); the source is kept at " + srcPath);
  if (wantRtc || (!onlyHipcc && (hipcc.empty() || access(hipcc.c_str(), X_OK) != 0))) {
    std::vector<char> image;
    if (std::string why = afir_target::compileWithHiprtc(source, &image); !why.empty())
      return Status::error((wantRtc ? std::string() : "hipcc not found (set HIPCC), and ") + why +
                           "; the source is kept at " + srcPath);
    std::ofstream f(objPath, std::ios::trunc | std::ios::binary);
    if (!f || !f.write(image.data(), (std::streamsize)image.size())) return Status::error("cannot write " + objPath);
    return objName;
  }
  std::vector<std::string> argv = {hipcc, "--genco"};
  for (const std::string &o : afir_target::regionCompileOptions()) argv.push_back(o);
  argv.insert(argv.end(), {"-o", objPath, srcPath});
  std::vector<char *> cargv;
  for (std::string &a : argv) cargv.push_back(a.data());
  cargv.push_back(nullptr);
  posix_spawn_file_actions_t actions;
  posix_spawn_file_actions_init(&actions);
  posix_spawn_file_actions_addopen(&actions, 1, logPath.c_str(), O_WRONLY | O_CREAT | O_TRUNC, 0644);
  posix_spawn_file_actions_adddup2(&actions, 1, 2);
  pid_t pid = 0;
  const int rc = posix_spawn(&pid, hipcc.c_str(), &actions, nullptr, cargv.data(), environ);
  posix_spawn_file_actions_destroy(&actions);
  if (rc != 0) return Status::error("cannot start " + hipcc + ": " + std::strerror(rc));
  int status = 0;
  while (waitpid(pid, &status, 0) < 0)
    if (errno != EINTR) return Status::error("waitpid failed for hipcc");
  if (!WIFEXITED(status) || WEXITSTATUS(status) != 0 || !fileExists(objPath)) {
    auto log = readTextFile(logPath);
    std::string tail = log ? *log : "";
    if (tail.size() > 1500) tail = tail.substr(tail.size() - 1500);
    return Status::error("hipcc rejected " + srcPath + ":\n" + tail);
  }
  std::remove(logPath.c_str());
  return objName;
}

Expected<HipKernelDescriptor> compileSourceText(const std::string &text, const std::string &nameHint) {
  HipKernelDescriptor d;
  // 1. an explicit request for a hand-tuned family
  for (const auto &kv : parseKeyValues(text))
    if (kv.first == "hip_kernel") {
      const KnownKernel *k = findKnown(kv.second);
      if (!k || kv.second == "fused_region") return Status::error("unknown hip_kernel: " + kv.second);
      d.hipKernel = kv.second;
      d.symbol = k->symbol;
      return d;
    }
  // 1b. a hand-written region program (the counterpart of the reference's
  // hand-written kernel sources, examples/real-npu-microcases/kernels/*.cpp)
  {
    size_t at = 0;
    while (at < text.size() && (text[at] == '#' || isspace((unsigned char)text[at]))) {
      if (text[at] == '#') while (at < text.size() && text[at] != '\n') ++at;
      else ++at;
    }
    if (text.compare(at, 15, "afir-hip-region") == 0) {
      afir_region::Program program;
      std::string why = afir_region::parse(text, &program);
      if (why.empty()) why = afir_region::validate(program);
      if (!why.empty()) return Status::error("invalid region program: " + why);
      d.kernelName = nameHint;
      d.hipKernel = "fused_region";
      d.symbol = findKnown("fused_region")->symbol;
      d.program = afir_region::serialize(program);
      return d;
    }
  }
  const std::string fn = firstFuncName(text);
  // 2. a function with an empty or opaque body that is named after a family
  // 3. MLIR text: translate the function to a region program
  if (text.find("func.func") != std::string::npos) {
    afir_target::Translation tr;
    const std::string why = afir_target::translateMlirToRegion(text, &tr);
    if (why.empty()) {
      d.kernelName = tr.functionName;
      d.hipKernel = "fused_region";
      d.symbol = findKnown("fused_region")->symbol;
      d.program = afir_region::serialize(tr.program);
      return d;
    }
    if (const KnownKernel *k = findKnown(fn)) {
      d.kernelName = fn;
      d.hipKernel = fn;
      d.symbol = k->symbol;
      return d;
    }
    return Status::error("cannot lower kernel source to a fused HIP kernel: " + why);
  }
  if (const KnownKernel *k = findKnown(nameHint)) {
    if (nameHint != "fused_region") {
      d.hipKernel = nameHint;
      d.symbol = k->symbol;
      return d;
    }
  }
  return Status::error("cannot map kernel source to a fused HIP kernel: expected MLIR text (func.func), a region program or "
                       "'hip_kernel=<family>' with one of fused_add_mul, broadcast_add_reducesum, "
                       "relu_broadcast_add_transpose, gather_scale_shift, matmul_add_leakyrelu");
}

Expected<KernelArtifact> compileArtifact(const CompileRequest &request) {
  if (request.kernelSource.empty()) return Status::error("kernel source is required");
  if (request.outputDir.empty()) return Status::error("output directory is required");
  auto text = readTextFile(request.kernelSource);
  if (!text) return Status::error("cannot read kernel source: " + request.kernelSource);
  auto compiled = compileSourceText(*text, request.kernelName);
  if (!compiled) return Status::error(compiled.error());
  const KnownKernel *known = findKnown(compiled->hipKernel);

  std::string name = request.kernelName;
  if (name.empty()) name = compiled->kernelName;
  if (name.empty()) name = firstFuncName(*text);
  if (name.empty()) name = compiled->hipKernel;

  if (!makeDirs(joinPath(request.outputDir, "out")))
    return Status::error("cannot create artifact manifest directory");

  HipKernelDescriptor d = *compiled;
  d.kernelName = name;
  d.library = defaultKernelLibraryPath();
  std::string codegenNote;
  if (!d.program.empty()) {
    // kernels specialised for the program; without them the interpreter
    // kernel of the library runs it
    auto object = compileRegionCodeObject(d.program, request.outputDir, name, request.emitOptions);
    if (object) {
      d.codeObject = *object;
      d.codeObjectDir = absolutePath(request.outputDir);
      d.codeObjectPreferred = !request.emitOptions.empty();
    } else if (!request.emitOptions.empty() && object.error().find("hipcc") == std::string::npos &&
               object.error().find("AFIR_HIP_CODEGEN") == std::string::npos) {
      return Status::error("emit options: " + object.error());   // asked-for choices must not be dropped silently
    } else {
      codegenNote = object.error();
    }
  }
  const std::string binRel = name + ".hipk";
  const std::string binPath = joinPath(request.outputDir, binRel);
  {
    std::ofstream f(binPath, std::ios::binary | std::ios::trunc);
    if (!f) return Status::error("cannot write artifact descriptor: " + binPath);
    f << serializeDescriptor(d);
  }
  KernelArtifact a;
  a.kernelName = name;
  a.kernelKind = request.kernelKind ? *request.kernelKind
                 : (d.program.find("\nmatmul ") != std::string::npos ? KernelKind::Mix : known->kind);
  a.regionProgram = d.program;
  a.codeObjectPath = resolveCodeObject(d, request.outputDir);
  a.codeObjectPreferred = d.codeObjectPreferred;
  a.codegenNote = codegenNote;
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
    if (!d.codeObject.empty()) f << "code_object_path=" << d.codeObject << "\n";
    if (!codegenNote.empty()) {
      std::string oneLine = codegenNote.substr(0, codegenNote.find('\n'));
      f << "code_object_note=" << oneLine << "\n";
    }
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
  a.regionProgram = d->program;
  a.codeObjectPath = resolveCodeObject(*d, root);
  a.codeObjectPreferred = d->codeObjectPreferred;
  a.codegenNote = kv["code_object_note"];
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
      auto task = v.getString("upstream_task");
      if (!task) return Status::error("missing required string field: upstream_task");
      auto output = v.getString("upstream_output");
      if (!output) return Status::error("missing required string field: upstream_output");
      b.fromTaskOutput = true;
      b.upstreamTask = *task;
      b.upstreamOutput = *output;
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
  if (auto v = root.getInteger("hip_grid")) {
    if (*v < 0 || *v > (1 << 30)) return Status::error("hip_grid must be between 0 and 2^30");
    spec.invocation.hipGrid = (int)*v;
  }
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
