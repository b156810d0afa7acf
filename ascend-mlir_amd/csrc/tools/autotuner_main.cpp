// autotuner for the HIP backend: searches the launch parameters a
// tiling_space.json leaves open, running every candidate on the GPU,
// validating it against the expected output and scoring it by kernel time.
// Same inputs, flags and best_config.json keys as the reference tool
// (tools/autotuner/autotuner_main.cpp:28-50 flags, :73-140 block_dim_expr,
// :557-595 best_config.json, :828-848 scoring), where the score is the
// simulator's wall clock; here it is the kernel's duration in nanoseconds
// from HIP events (best of --repeats launches).
//
//   autotuner --space tiling_space.json (--kernel K.mlir | --artifact-root DIR)
//             --inputs a.npy,b.npy --expected e.npy --shape M=32,N=32
//             [--output best_config.json] [--kernel-kind vec|cube|mix] [--soc S]
//             [--atol A] [--rtol R] [--repeats N] [--buffer-sets N] [--ramp-ms MS] [--device N]
//
// tiling_space.json: {"kernel", "kernel_file", "soc", "block_dim_expr",
//   "block_dim_values": [..] (this backend: explicit grid sizes to try, 0 =
//   the launcher's own choice), "tiling_params": [{"name", "type",
//   "values": [..] | "min","max","step" | "fixed": true + "shape_key" | "value"}]}.
// A parameter named dim_arg<A>_<D> with nothing else given takes dimension D
// of argument A from the .npy files (inputs first, then the expected output).
// A parameter named emit_tile_p / emit_tile_q / emit_unroll is a compile-time
// choice of the emitted kernels (only with --kernel): every combination is
// compiled into its own artifact under the build directory and is not part of
// the TilingData bytes.
//
// A parameter named build_<MACRO> is a compile-time choice of the hand-tuned
// kernels (tile shapes, rings, grids: the AFIR_* macros of csrc/kernels): every
// combination is built into a kernel library of its own under the build
// directory (python3 build.py --variant ... -DMACRO=value, beside this tool's
// bin/ directory; needs hipcc) and the candidate is launched from that library.
// Like emit_* it is not part of the TilingData bytes.
//
// A parameter named env_<NAME> is a launch-time choice of the hand-tuned kernels
// that they read from the environment (the AFIR_*_PHASE_GBS / _BASE_NS holds of
// the kernels that separate reads from writes): the candidate runs with NAME set
// to the value, in this process and from the one shipped library.  Not part of
// the TilingData bytes either.
//
// Exit codes: 0 ok, 1 no candidate passed, 2 run error, 4 bad invocation.
#include <cctype>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <map>
#include <sstream>
#include <string>
#include <vector>

#include <unistd.h>

#include "../runtime/runtime.h"

namespace {

using namespace afirt;

// Directory of this executable (bin/), for the build script beside it.
std::string toolDirectory() {
  char buf[4096];
  const ssize_t n = readlink("/proc/self/exe", buf, sizeof buf - 1);
  if (n <= 0) return ".";
  buf[n] = 0;
  std::string path(buf);
  const size_t slash = path.rfind('/');
  return slash == std::string::npos ? "." : path.substr(0, slash);
}

struct Param {
  std::string name, type = "int64", shapeKey;
  bool fixed = false, hasValue = false;
  int64_t value = 0;
  std::vector<int64_t> values;   // search candidates (empty = not searched)
};

// Testing-only runner (--testing-driver=hip-success): no device, outputs stay
// zero, and the reported kernel time shrinks with block_dim so that a search
// has a defined winner; AFIR_TESTING_EXTRA_US in the environment is added to it
// (what an env_* parameter looks like to a kernel that reads it).
class TestingRunner final : public ExecutionRunner {
 public:
  ExecutionRunnerMode mode() const override { return ExecutionRunnerMode::Simulation; }
  Status initialize(int) override { return Status::success(); }
  Status runFile(const FileExecutionLaunch &, RunArgs &) override { return Status::success(); }
  Status runDynamicLibraryArtifact(const DynamicLibraryExecutionLaunch &, RunArgs &args) override {
    us_ = 1000.0 / (1 + args.block_dim);
    if (const char *extra = getenv("AFIR_TESTING_EXTRA_US")) us_ += std::atof(extra);
    return Status::success();
  }
  double lastKernelMicroseconds() const override { return us_; }

 private:
  double us_ = -1.0;
};

std::vector<std::string> split(const std::string &s, char sep) {
  std::vector<std::string> out;
  std::istringstream ss(s);
  for (std::string t; std::getline(ss, t, sep);)
    if (!t.empty()) out.push_back(t);
  return out;
}

// "ceil(X / Y)", "X / Y", "X", integers; X, Y are parameter or shape names
// (tools/autotuner/autotuner_main.cpp:73-140).
bool evalBlockDimExpr(std::string expr, const std::map<std::string, int64_t> &vars, int64_t *out,
                      std::string *why) {
  std::string e;
  for (char c : expr)
    if (!isspace((unsigned char)c)) e += c;
  bool ceil = false;
  if (e.compare(0, 5, "ceil(") == 0 && e.back() == ')') {
    ceil = true;
    e = e.substr(5, e.size() - 6);
  }
  auto term = [&](const std::string &t, int64_t *v) {
    if (t.empty()) return false;
    char *end = nullptr;
    long long n = std::strtoll(t.c_str(), &end, 10);
    if (!*end) { *v = n; return true; }
    auto it = vars.find(t);
    if (it == vars.end()) { *why = "unknown name '" + t + "' in block_dim_expr"; return false; }
    *v = it->second;
    return true;
  };
  const size_t slash = e.find('/');
  int64_t a = 0, b = 1;
  if (!term(slash == std::string::npos ? e : e.substr(0, slash), &a)) return false;
  if (slash != std::string::npos && !term(e.substr(slash + 1), &b)) return false;
  if (b <= 0) { *why = "block_dim_expr divides by a non-positive value"; return false; }
  *out = ceil ? (a + b - 1) / b : a / b;
  return true;
}

std::string jsonEscape(const std::string &s) {
  std::string o;
  for (char c : s) {
    if (c == '"' || c == '\\') o += '\\';
    o += c;
  }
  return o;
}

int usage(const char *msg) {
  std::fprintf(stderr, "Error: %s\n", msg);
  std::fprintf(stderr,
               "usage: autotuner --space S.json (--kernel K.mlir | --artifact-root DIR) --inputs a.npy,b.npy "
               "--expected e.npy --shape M=32,N=32 [--output best_config.json] [--repeats N]\n");
  return 4;
}

}  // namespace

int main(int argc, char **argv) {
  std::map<std::string, std::string> opt;
  for (int i = 1; i < argc; ++i) {
    std::string a = argv[i];
    if (a.rfind("--", 0) == 0) a = a.substr(2);
    else if (a.rfind("-", 0) == 0) a = a.substr(1);
    else return usage(("unexpected argument '" + std::string(argv[i]) + "'").c_str());
    const size_t eq = a.find('=');
    if (eq != std::string::npos) opt[a.substr(0, eq)] = a.substr(eq + 1);
    else if (i + 1 < argc) opt[a] = argv[++i];
    else return usage(("option '--" + a + "' requires a value").c_str());
  }
  for (const char *req : {"space", "inputs", "expected", "shape"})
    if (!opt.count(req)) return usage((std::string("--") + req + " is required").c_str());
  if (opt.count("kernel") == opt.count("artifact-root"))
    return usage("provide exactly one of --kernel or --artifact-root");

  // ---- tiling space ----
  auto text = readTextFile(opt["space"]);
  if (!text) return usage(("cannot read " + opt["space"]).c_str());
  auto json = parseJson(*text);
  if (!json || json->kind != Json::Object) return usage("tiling space is not a JSON object");
  const Json *params = json->getArray("tiling_params");
  if (!params) return usage("tiling space: missing 'tiling_params' array");
  std::vector<Param> space;
  for (const Json &p : params->array) {
    Param q;
    auto name = p.getString("name");
    if (!name) return usage("tiling space: parameter without a name");
    q.name = *name;
    q.type = p.getString("type").value_or("int64");
    q.shapeKey = p.getString("shape_key").value_or("");
    q.fixed = p.getBoolean("fixed").value_or(false);
    if (auto v = p.getInteger("value")) { q.hasValue = true; q.value = *v; }
    if (const Json *vals = p.getArray("values")) {
      for (const Json &v : vals->array)
        if (v.kind == Json::Number) q.values.push_back(v.is_integer ? v.integer : (int64_t)v.number);
    } else if (p.getInteger("min") && p.getInteger("max")) {
      const int64_t lo = *p.getInteger("min"), hi = *p.getInteger("max");
      const int64_t step = p.getInteger("step").value_or(1);
      if (step <= 0 || hi < lo) return usage(("bad range of parameter " + q.name).c_str());
      for (int64_t v = lo; v <= hi; v += step) q.values.push_back(v);
    }
    space.push_back(q);
  }
  std::vector<int64_t> blockDims;
  if (const Json *b = json->getArray("block_dim_values"))
    for (const Json &v : b->array)
      if (v.kind == Json::Number && v.is_integer && v.integer >= 0) blockDims.push_back(v.integer);
  const std::string blockDimExpr = json->getString("block_dim_expr").value_or("");

  std::map<std::string, int64_t> shape;
  for (const std::string &kv : split(opt["shape"], ',')) {
    const size_t eq = kv.find('=');
    if (eq == std::string::npos) return usage(("bad --shape entry '" + kv + "'").c_str());
    shape[kv.substr(0, eq)] = std::strtoll(kv.c_str() + eq + 1, nullptr, 10);
  }

  // ---- artifact ----
  KernelArtifact artifact;
  CompileRequest baseRequest;
  if (opt.count("artifact-root")) {
    auto a = loadArtifactFromRoot(opt["artifact-root"]);
    if (!a) return usage(a.error().c_str());
    artifact = *a;
  } else {
    CompileRequest req;
    req.kernelSource = opt["kernel"];
    req.outputDir = opt.count("build-dir") ? opt["build-dir"] : opt["space"] + ".artifact";
    req.kernelName = json->getString("kernel").value_or("");
    req.socVersion = opt.count("soc") ? opt["soc"] : json->getString("soc").value_or("gfx950");
    if (opt.count("kernel-kind")) {
      auto kind = parseKernelKind(opt["kernel-kind"]);
      if (!kind) return usage(kind.error().c_str());
      req.kernelKind = *kind;
    }
    auto a = compileArtifact(req);
    if (!a) return usage(a.error().c_str());
    artifact = *a;
    baseRequest = req;
  }

  // ---- tensors ----
  RunArgs base;
  std::vector<std::vector<int64_t>> argShapes;
  for (const std::string &path : split(opt["inputs"], ',')) {
    auto arr = LoadNpy(path);
    if (!arr) return usage(arr.error().c_str());
    argShapes.push_back(arr->shape);
    base.inputs.push_back(std::move(*arr));
  }
  auto expected = LoadNpy(opt["expected"]);
  if (!expected) return usage(expected.error().c_str());
  argShapes.push_back(expected->shape);

  // ---- resolve fixed parameters, collect search variables ----
  std::map<std::string, int64_t> fixedValues;
  std::vector<const Param *> search;
  for (const Param &p : space) {
    if (!p.shapeKey.empty()) {
      auto it = shape.find(p.shapeKey);
      if (it == shape.end()) return usage(("shape key '" + p.shapeKey + "' of parameter " + p.name + " is not in --shape").c_str());
      fixedValues[p.name] = it->second;
    } else if (p.hasValue) {
      fixedValues[p.name] = p.value;
    } else if (p.values.size() == 1) {
      fixedValues[p.name] = p.values[0];
    } else if (!p.values.empty()) {
      search.push_back(&p);
    } else {
      int a = -1, d = -1;
      if (std::sscanf(p.name.c_str(), "dim_arg%d_%d", &a, &d) == 2 && a >= 0 && a < (int)argShapes.size() &&
          d >= 0 && d < (int)argShapes[a].size())
        fixedValues[p.name] = argShapes[a][d];
      else
        return usage(("parameter '" + p.name + "' has no shape_key, value or candidates").c_str());
    }
  }
  std::vector<std::map<std::string, int64_t>> combos(1);
  for (const Param *p : search) {
    std::vector<std::map<std::string, int64_t>> next;
    for (const auto &c : combos)
      for (int64_t v : p->values) {
        auto e = c;
        e[p->name] = v;
        next.push_back(std::move(e));
      }
    combos = std::move(next);
  }

  const bool testing = opt.count("testing-driver") && opt["testing-driver"] == "hip-success";
  if (opt.count("testing-driver") && !testing) return usage("unsupported testing driver");
  std::unique_ptr<ExecutionRunner> runner =
      testing ? std::unique_ptr<ExecutionRunner>(new TestingRunner()) : createHipExecutionRunner();
  if (Status st = runner->initialize(opt.count("device") ? std::atoi(opt["device"].c_str()) : 0); !st.ok()) {
    std::fprintf(stderr, "Error: [hip:executor_initialize] %s\n", st.message.c_str());
    return 2;
  }
  const double atol = opt.count("atol") ? std::atof(opt["atol"].c_str()) : 1.0;
  const double rtol = opt.count("rtol") ? std::atof(opt["rtol"].c_str()) : 1e-2;
  const int repeats = opt.count("repeats") ? std::max(1, std::atoi(opt["repeats"].c_str())) : 5;
  // --buffer-sets N: the timed launches of a candidate rotate over N copies of its tensors on the
  // device, so that repeated launches are not served from the last-level cache
  const int bufferSets = opt.count("buffer-sets") ? std::max(1, std::atoi(opt["buffer-sets"].c_str())) : 1;
  // --ramp-ms MS: each candidate is launched back to back for MS milliseconds before its timed
  // launches, which then run without synchronisations in between (the device's sustained clocks)
  const double rampMs = opt.count("ramp-ms") ? std::max(0.0, std::atof(opt["ramp-ms"].c_str())) : 0.0;

  DynamicLibraryExecutionLaunch launch;
  launch.sharedLibraryPath = artifact.sharedLibraryPath;
  launch.symbolName = artifact.sharedLibrarySymbol;
  launch.regionProgram = artifact.regionProgram;
  launch.codeObjectPath = artifact.codeObjectPath;

  struct Best {
    bool found = false;
    double ns = 0, maxAbs = 0;
    int64_t blockDim = 0;
    std::map<std::string, int64_t> config;
    KernelArtifact artifact;
  } best;
  size_t index = 0, total = 0;
  for (const auto &c : combos) {
    (void)c;
    total += blockDims.empty() ? 1 : blockDims.size();
  }
  for (const auto &combo : combos) {
    std::map<std::string, int64_t> vars = fixedValues;
    for (const auto &kv : combo) vars[kv.first] = kv.second;
    std::vector<int64_t> dims = blockDims;
    if (dims.empty()) {
      int64_t bd = 0;
      if (!blockDimExpr.empty()) {
        auto all = vars;
        for (const auto &kv : shape) all.emplace(kv.first, kv.second);
        std::string why;
        if (!evalBlockDimExpr(blockDimExpr, all, &bd, &why)) return usage(why.c_str());
      }
      dims.push_back(bd);
    }
    // tiling bytes in the order of the space
    std::vector<TilingField> fields;
    std::vector<std::pair<std::string, int64_t>> values;
    std::map<std::string, int64_t> emitOptions, buildMacros, envValues;
    for (const Param &p : space) {
      if (p.name.rfind("env_", 0) == 0) {
        envValues[p.name.substr(4)] = vars[p.name];
        continue;
      }
      if (p.name.rfind("emit_", 0) == 0) {
        emitOptions[p.name.substr(5)] = vars[p.name];
        continue;
      }
      if (p.name.rfind("build_", 0) == 0) {
        buildMacros[p.name.substr(6)] = vars[p.name];
        continue;
      }
      fields.push_back({p.name, p.type});
      values.push_back({p.name, vars[p.name]});
    }
    // kernels emitted with these choices: one artifact per combination
    KernelArtifact candidateArtifact = artifact;
    if (!emitOptions.empty()) {
      if (baseRequest.kernelSource.empty())
        return usage("emit_* parameters need --kernel (the kernels are compiled per candidate)");
      CompileRequest req = baseRequest;
      req.emitOptions = emitOptions;
      req.outputDir = baseRequest.outputDir + "/emit";
      for (const auto &kv : emitOptions) req.outputDir += "_" + kv.first + std::to_string(kv.second);
      auto a = compileArtifact(req);
      if (!a) {
        for (int64_t bd : dims) {
          ++index;
          std::printf("[%zu/%zu]", index, total);
          for (const auto &kv : combo) std::printf(" %s=%lld", kv.first.c_str(), (long long)kv.second);
          std::printf(" block_dim=%lld ... FAIL  %s\n", (long long)bd, a.error().c_str());
        }
        continue;
      }
      candidateArtifact = *a;
    }
    // hand-tuned kernels built with these choices: one kernel library per combination
    if (!buildMacros.empty() && !testing) {
      const std::string variantDir = !baseRequest.outputDir.empty() ? baseRequest.outputDir
                                     : opt.count("build-dir")        ? opt["build-dir"]
                                                                     : opt["space"] + ".artifact";
      std::string lib = variantDir + "/variant";
      std::string flags;
      for (const auto &kv : buildMacros) {
        for (char ch : kv.first)
          if (!(std::isalnum((unsigned char)ch) || ch == '_')) return usage("build_* parameter names must be macro names");
        lib += "_" + kv.first + std::to_string(kv.second);
        flags += " -D" + kv.first + "=" + std::to_string(kv.second);
      }
      lib += ".so";
      if (!std::ifstream(lib).good()) {
        const std::string cmd = "mkdir -p '" + variantDir + "' && python3 '" + toolDirectory() +
                                "/../build.py' --variant '" + lib + "'" + flags + " > '" + lib + ".log' 2>&1";
        if (std::system(cmd.c_str()) != 0) {
          for (int64_t bd : dims) {
            ++index;
            std::printf("[%zu/%zu]", index, total);
            for (const auto &kv : combo) std::printf(" %s=%lld", kv.first.c_str(), (long long)kv.second);
            std::printf(" block_dim=%lld ... FAIL  the kernel library does not build with these choices (%s.log)\n",
                        (long long)bd, lib.c_str());
          }
          continue;
        }
      }
      candidateArtifact.sharedLibraryPath = lib;
    }
    launch.sharedLibraryPath = candidateArtifact.sharedLibraryPath;
    launch.symbolName = candidateArtifact.sharedLibrarySymbol;
    launch.regionProgram = candidateArtifact.regionProgram;
    launch.codeObjectPath = candidateArtifact.codeObjectPath;
    launch.preferCodeObject = candidateArtifact.codeObjectPreferred;
    auto packed = TilingSchema::fromFields(fields).pack(values);
    if (!packed) return usage(packed.error().c_str());
    // launch-time choices read from the environment: set for this combination's runs
    struct EnvGuard {
      std::vector<std::string> names;
      ~EnvGuard() { for (const std::string &n : names) unsetenv(n.c_str()); }
    } envGuard;
    for (const auto &kv : envValues) {
      for (char ch : kv.first)
        if (!(std::isalnum((unsigned char)ch) || ch == '_')) return usage("env_* parameter names must be variable names");
      setenv(kv.first.c_str(), std::to_string(kv.second).c_str(), 1);
      envGuard.names.push_back(kv.first);
    }

    for (int64_t bd : dims) {
      ++index;
      std::printf("[%zu/%zu]", index, total);
      for (const auto &kv : combo) std::printf(" %s=%lld", kv.first.c_str(), (long long)kv.second);
      std::printf(" block_dim=%lld ...", (long long)bd);
      std::fflush(stdout);
      RunArgs args;
      args.tiling = *packed;
      args.block_dim = (int)bd;
      args.hip_grid = (int)bd;     // a candidate's block_dim is a HIP grid here, not an AI-core count
      args.inputs.resize(base.inputs.size());
      for (size_t i = 0; i < base.inputs.size(); ++i) {
        args.inputs[i].shape = base.inputs[i].shape;
        args.inputs[i].dtype = base.inputs[i].dtype;
        args.inputs[i].setExternal(base.inputs[i].data);
      }
      NDArray out;
      out.shape = expected->shape;
      out.dtype = expected->dtype;
      out.allocate();
      args.outputs.push_back(std::move(out));
      // one run: the kernel is launched 1 + (repeats - 1) times on the same device buffers
      double bestNs = -1;
      args.timing_repeats = repeats - 1;
      args.buffer_sets = bufferSets;
      args.ramp_ms = rampMs;
      Status st = runner->runDynamicLibraryArtifact(launch, args);
      const double us = runner->lastKernelMicroseconds();
      if (st.ok() && us >= 0) bestNs = us * 1e3;
      if (!st.ok()) {
        std::printf(" FAIL  %s\n", st.message.c_str());
        continue;
      }
      std::vector<NDArray> exp(1);
      exp[0].shape = expected->shape;
      exp[0].dtype = expected->dtype;
      exp[0].setExternal(expected->data);
      auto cmp = compareRuntimeOutputs(args.outputs, exp, atol, rtol);
      if (!cmp || (!cmp->passed && !testing)) {
        std::printf(" FAIL  %s\n", cmp ? cmp->errorMessage.c_str() : cmp.error().c_str());
        continue;
      }
      std::printf(" OK  score=%.0f max_abs_diff=%g\n", bestNs, cmp->maxAbsDiff);
      if (!best.found || bestNs < best.ns) {
        best.artifact = candidateArtifact;
        best.found = true;
        best.ns = bestNs;
        best.maxAbs = cmp->maxAbsDiff;
        best.blockDim = bd;
        best.config = vars;
      }
    }
  }
  if (!best.found) {
    std::fprintf(stderr, "Error: no candidate passed validation\n");
    return 1;
  }

  const std::string outPath = opt.count("output") ? opt["output"] : "best_config.json";
  std::ofstream f(outPath, std::ios::trunc);
  if (!f) {
    std::fprintf(stderr, "Error: cannot write best-config JSON: %s\n", outPath.c_str());
    return 2;
  }
  f << "{\n";
  f << "  \"kernel_name\": \"" << jsonEscape(best.artifact.kernelName) << "\",\n";
  f << "  \"kernel_type\": \"" << kernelKindName(best.artifact.kernelKind) << "\",\n";
  f << "  \"soc\": \"" << jsonEscape(best.artifact.socVersion) << "\",\n";
  f << "  \"artifact_root\": \"" << jsonEscape(best.artifact.artifactRoot) << "\",\n";
  f << "  \"manifest_path\": \"" << jsonEscape(best.artifact.manifestPath) << "\",\n";
  f << "  \"device_binary_path\": \"" << jsonEscape(best.artifact.deviceBinaryPath) << "\",\n";
  f << "  \"kernel_file\": \"" << jsonEscape(json->getString("kernel_file").value_or("")) << "\",\n";
  f << "  \"best\": {\"block_dim\": " << best.blockDim << ", \"cycle_count\": " << (long long)std::llround(best.ns)
    << ", \"score\": " << (long long)std::llround(best.ns) << ", \"score_unit\": \"ns\", \"max_abs_diff\": "
    << best.maxAbs << "},\n";
  f << "  \"config\": {";
  bool first = true;
  for (const auto &kv : best.config) {
    f << (first ? "" : ", ") << "\"" << jsonEscape(kv.first) << "\": " << kv.second;
    first = false;
  }
  f << "},\n  \"shape\": {";
  first = true;
  for (const auto &kv : shape) {
    f << (first ? "" : ", ") << "\"" << jsonEscape(kv.first) << "\": " << kv.second;
    first = false;
  }
  f << "},\n  \"candidates\": " << total << "\n}\n";
  std::printf("best: block_dim=%lld score=%.0f ns -> %s\n", (long long)best.blockDim, best.ns, outPath.c_str());
  return 0;
}
