// runtime-session for the HIP backend: same flags, printed keys and exit codes
// as the reference CLI (tools/runtime-session/runtime_session_main.cpp:31-92,
// 133-194, 244-397): 0 = ok, 2 = run/plan error, 4 = bad invocation.
//
//   runtime-session --kernel K.mlir --output DIR [--name N] [--kernel-kind vec|cube|mix] [--soc S]
//   runtime-session --artifact-root DIR [--run]
//   runtime-session --run-manifest M.json --run [--device N]
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <sstream>
#include <string>

#include "../runtime/runtime.h"

namespace {

using namespace afirt;

// Testing-only runner: succeeds without a device and leaves the outputs zero
// (the reference has the same kind of hidden driver, --testing-driver=npu-success).
class SuccessfulTestingRunner final : public ExecutionRunner {
 public:
  ExecutionRunnerMode mode() const override { return ExecutionRunnerMode::Simulation; }
  Status initialize(int) override { return Status::success(); }
  Status runFile(const FileExecutionLaunch &, RunArgs &) override { return Status::success(); }
  Status runDynamicLibraryArtifact(const DynamicLibraryExecutionLaunch &, RunArgs &args) override {
    // the grid rule of the HIP runner, without a launch: "hip_grid" is a grid, block_dim is not
    grid_.kernel = "testing";
    grid_.source = args.hip_grid > 0 ? "hip_grid" : "launcher";
    grid_.workgroups = args.hip_grid > 0 ? (uint32_t)args.hip_grid : 2048u;
    grid_.threads = 256;
    return Status::success();
  }
  double lastKernelMicroseconds() const override { return 12.5; }   // a fixed figure for the profile tests
  LaunchedGrid lastLaunchedGrid() const override { return grid_; }

 private:
  LaunchedGrid grid_;
};
std::unique_ptr<ExecutionRunner> makeTestingRunner() {
  return std::make_unique<SuccessfulTestingRunner>();
}

void printErrorSummary(const SessionSummary &s) {
  std::fprintf(stderr, "session.backend=%s\n", s.backend.c_str());
  std::fprintf(stderr, "session.result=error\n");
  if (s.validationRan && s.errorStage == "validate") std::fprintf(stderr, "session.validation=fail\n");
  if (!s.errorStage.empty()) std::fprintf(stderr, "session.error_stage=%s\n", s.errorStage.c_str());
  std::fprintf(stderr, "session.error=%s\n", s.errorMessage.c_str());
  std::fprintf(stderr, "Error: %s\n", s.rawErrorMessage.c_str());
}

}  // namespace

int main(int argc, char **argv) {
  std::map<std::string, std::string> opt;
  bool run = false;
  const char *valued[] = {"emit-options", "kernel", "kernel-kind", "output", "name", "soc", "artifact-root",
                          "run-manifest", "task-id", "testing-driver", "device", "cann-mlir",
                          "npy-dir"};
  for (int i = 1; i < argc; ++i) {
    std::string a = argv[i];
    if (a.rfind("--", 0) == 0) a = a.substr(2);
    else if (a.rfind("-", 0) == 0) a = a.substr(1);
    else {
      std::fprintf(stderr, "Error: unexpected argument '%s'\n", argv[i]);
      return 4;
    }
    std::string key = a, value;
    bool hasValue = false;
    size_t eq = a.find('=');
    if (eq != std::string::npos) {
      key = a.substr(0, eq);
      value = a.substr(eq + 1);
      hasValue = true;
    }
    if (key == "run") {
      run = !hasValue || value == "true" || value == "1";
      continue;
    }
    if (key == "help" || key == "h") {
      std::printf("task graph runtime planning and execution CLI for artifacts and session graphs (HIP backend)\n"
                  "  --kernel <file> --output <dir> [--name N] [--kernel-kind vec|cube|mix] [--soc S]\n"
                  "           [--emit-options tile_p=64,tile_q=64,unroll=0]\n"
                  "  --artifact-root <dir>\n  --run-manifest <json>\n  --run\n  --device <n>\n");
      return 0;
    }
    bool known = false;
    for (const char *v : valued) known = known || key == v;
    if (!known) {
      std::fprintf(stderr, "Error: unknown option '--%s'\n", key.c_str());
      return 4;
    }
    if (!hasValue) {
      if (i + 1 >= argc) {
        std::fprintf(stderr, "Error: option '--%s' requires a value\n", key.c_str());
        return 4;
      }
      value = argv[++i];
    }
    opt[key] = value;
  }

  RunTaskSpec task;
  RunManifestSpec session;   // every task of the manifest (or the one implied by the flags)
  task.taskId = opt.count("task-id") ? opt["task-id"] : "main";
  std::string backend = "hip";
  if (opt.count("run-manifest")) {
    auto manifest = loadRunManifest(opt["run-manifest"]);
    if (!manifest) {
      std::fprintf(stderr, "Error: %s\n", manifest.error().c_str());
      return 4;
    }
    if (manifest->backend != "hip")
      std::printf("session.backend_requested=%s\n", manifest->backend.c_str());
    session = *manifest;
    task = manifest->tasks[0];
  } else {
    const bool hasRoot = opt.count("artifact-root") != 0, hasKernel = opt.count("kernel") != 0;
    if (hasRoot == hasKernel) {
      std::fprintf(stderr, "Error: provide exactly one of --artifact-root or --kernel\n");
      return 4;
    }
    KernelArtifact artifact;
    if (hasRoot) {
      auto loaded = loadArtifactFromRoot(opt["artifact-root"]);
      if (!loaded) {
        std::fprintf(stderr, "Error: %s\n", loaded.error().c_str());
        return 4;
      }
      artifact = *loaded;
    } else {
      CompileRequest req;
      req.kernelSource = opt["kernel"];
      req.outputDir = opt.count("output") ? opt["output"] : "./build/runtime-session-artifact";
      req.kernelName = opt.count("name") ? opt["name"] : "";
      req.socVersion = opt.count("soc") ? opt["soc"] : "gfx950";
      if (opt.count("emit-options")) {   // --emit-options tile_p=64,tile_q=128,unroll=2
        std::istringstream items(opt["emit-options"]);
        for (std::string kv; std::getline(items, kv, ',');) {
          const size_t eq = kv.find('=');
          if (eq == std::string::npos || eq == 0) {
            std::fprintf(stderr, "Error: --emit-options takes name=value pairs, got '%s'\n", kv.c_str());
            return 4;
          }
          req.emitOptions[kv.substr(0, eq)] = std::strtoll(kv.c_str() + eq + 1, nullptr, 10);
        }
      }
      if (opt.count("kernel-kind")) {
        auto kind = parseKernelKind(opt["kernel-kind"]);
        if (!kind) {
          std::fprintf(stderr, "Error: %s\n", kind.error().c_str());
          return 4;
        }
        req.kernelKind = *kind;
      }
      auto compiled = compileArtifact(req);
      if (!compiled) {
        std::fprintf(stderr, "Error: %s\n", compiled.error().c_str());
        return 4;
      }
      artifact = *compiled;
    }
    std::printf("artifact.kernel_name=%s\n", artifact.kernelName.c_str());
    std::printf("artifact.root=%s\n", artifact.artifactRoot.c_str());
    std::printf("artifact.manifest=%s\n", artifact.manifestPath.c_str());
    std::printf("artifact.soc=%s\n", artifact.socVersion.c_str());
    task.artifactRoot = artifact.artifactRoot;
  }

  RunnerFactory factory = nullptr;
  if (opt.count("testing-driver")) {
    if (opt["testing-driver"] != "hip-success") {
      std::fprintf(stderr, "Error: unsupported testing driver: %s\n", opt["testing-driver"].c_str());
      return 4;
    }
    factory = &makeTestingRunner;
  }

  if (session.tasks.empty()) session.tasks.push_back(task);
  auto plan = planTasks(session);
  if (!plan) {
    std::fprintf(stderr, "Error: %s\n", plan.error().c_str());
    return 4;
  }
  std::printf("session.plan.tasks=%zu\n", plan->size());
  for (size_t i = 0; i < plan->size(); ++i)
    std::printf("session.plan[%zu]=%s\n", i, session.tasks[(*plan)[i]].taskId.c_str());
  std::fflush(stdout);
  if (!run) return 0;

  if (!opt.count("run-manifest")) {
    std::fprintf(stderr, "session.backend=%s\nsession.result=error\n", backend.c_str());
    std::fprintf(stderr, "session.error_stage=bindings\n");
    std::fprintf(stderr, "session.error=running needs tensor bindings: use --run-manifest\n");
    std::fprintf(stderr, "Error: [hip:bindings] running needs tensor bindings: use --run-manifest\n");
    return 2;
  }

  const int device = opt.count("device") ? std::atoi(opt["device"].c_str()) : 0;
  // outputs without a path go to a directory next to the manifest
  std::string workdir = opt["run-manifest"];
  const size_t slash = workdir.rfind('/');
  workdir = slash == std::string::npos ? "." : workdir.substr(0, slash);
  SessionSummary s = runSession(session, factory, device, workdir);
  if (!s.success) {
    printErrorSummary(s);
    return 2;
  }
  std::printf("session.backend=%s\n", s.backend.c_str());
  std::printf("session.result=success\n");
  if (s.validationRan && s.validationPassed) std::printf("session.validation=pass\n");
  if (!s.profileArtifacts.empty()) {
    // profiles outlive the run directory: <tmp>/ascendc-runtime-profiles/<session id>/
    // (tools/runtime-session/runtime_session_main.cpp:212-228)
    const char *tmp = std::getenv("TMPDIR");
    const std::string root = std::string(tmp && *tmp ? tmp : "/tmp") + "/ascendc-runtime-profiles";
    if (Status st = retainProfileArtifacts(s, root); !st.ok()) {
      s.success = false;
      s.errorStage = "profiling";
      s.errorMessage = st.message;
      s.rawErrorMessage = "[hip:profiling] " + st.message;
      printErrorSummary(s);
      return 2;
    }
  }
  std::printf("session.profile.session_id=%s\n", s.sessionId.c_str());
  std::printf("session.profile.count=%zu\n", s.profileArtifacts.size());
  for (size_t i = 0; i < s.profileArtifacts.size(); ++i)
    std::printf("session.profile[%zu]=%s\n", i, s.profileArtifacts[i].path.c_str());
  if (!s.retainedSummaryPath.empty()) std::printf("session.profile.summary=%s\n", s.retainedSummaryPath.c_str());
  if (s.validationRan) {
    std::printf("session.runtime.attribute.max_abs_diff=%g\n", s.comparison.maxAbsDiff);
    std::printf("session.runtime.attribute.mean_abs_diff=%g\n", s.comparison.meanAbsDiff);
  }
  for (const auto &kv : s.runtimeAttributes)
    std::printf("session.runtime.attribute.%s=%s\n", kv.first.c_str(), kv.second.c_str());
  for (const auto &kv : s.runtimeCounters)
    std::printf("session.runtime.counter.%s=%lld\n", kv.first.c_str(), (long long)kv.second);
  return 0;
}
