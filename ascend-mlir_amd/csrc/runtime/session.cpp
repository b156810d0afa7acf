// Single-task session: the run sequence of the reference's backend
// (lib/Runtime/Execution/SimBackend.cpp:240-304,387-486) on the HIP runner:
// load artifact -> pack tiling -> load input .npy -> allocate outputs from the
// expected shapes -> launch -> compare -> save outputs.  Errors carry the
// stage they happened in, as "[hip:<stage>] message".
#include "runtime.h"

namespace afirt {

namespace {

SessionSummary fail(SessionSummary s, const char *stage, const std::string &msg) {
  s.success = false;
  s.errorStage = stage;
  s.errorMessage = msg;
  s.rawErrorMessage = std::string("[hip:") + stage + "] " + msg;
  return s;
}

}  // namespace

SessionSummary runSingleTask(const RunTaskSpec &task, RunnerFactory factory, int deviceId) {
  SessionSummary summary;
  const ExecutionInvocation &inv = task.invocation;
  summary.validationRan = !inv.expectedOutputs.empty();

  // ---- artifact ----
  auto artifact = loadArtifactFromRoot(task.artifactRoot);
  if (!artifact) return fail(summary, "artifact", artifact.error());
  summary.runtimeAttributes["kernel_name"] = artifact->kernelName;
  summary.runtimeAttributes["launch_symbol"] = artifact->sharedLibrarySymbol;

  // ---- bindings ----
  RunArgs args;
  args.block_dim = inv.blockDim;
  args.workspace_size = inv.workspaceSize;
  auto tiling = packTilingBytes(inv.tiling);
  if (!tiling) return fail(summary, "bindings", tiling.error());
  args.tiling = std::move(*tiling);

  for (const TensorBinding &b : inv.inputs) {
    if (b.path.empty()) return fail(summary, "bindings", "input '" + b.name + "' has no path");
    auto arr = LoadNpy(b.path);
    if (!arr) return fail(summary, "bindings", arr.error());
    if (!b.shape.empty() && b.shape != arr->shape)
      return fail(summary, "bindings", "input '" + b.name + "' shape does not match " + b.path);
    if (b.dtype && *b.dtype != arr->dtype)
      return fail(summary, "bindings", "input '" + b.name + "' dtype does not match " + b.path);
    args.inputs.push_back(std::move(*arr));
  }

  std::vector<NDArray> expected;
  for (const TensorBinding &b : inv.expectedOutputs) {
    auto arr = LoadNpy(b.path);
    if (!arr) return fail(summary, "bindings", arr.error());
    expected.push_back(std::move(*arr));
  }
  if (inv.outputs.empty()) return fail(summary, "bindings", "at least one output binding is required");
  if (!expected.empty() && expected.size() != inv.outputs.size())
    return fail(summary, "bindings",
                format("expected output metadata mismatch: %zu outputs, %zu expected outputs",
                       inv.outputs.size(), expected.size()));
  for (size_t i = 0; i < inv.outputs.size(); ++i) {
    const TensorBinding &b = inv.outputs[i];
    NDArray out;
    if (!b.shape.empty() && b.dtype) {
      out.shape = b.shape;
      out.dtype = *b.dtype;
      if (!expected.empty() && (expected[i].shape != out.shape || expected[i].dtype != out.dtype))
        return fail(summary, "bindings",
                    "expected output metadata mismatch for output '" + b.name + "'");
    } else if (!expected.empty()) {
      out.shape = expected[i].shape;
      out.dtype = expected[i].dtype;
    } else {
      return fail(summary, "bindings",
                  "output '" + b.name + "' needs shape and dtype (or an expected output to take them from)");
    }
    out.allocate();
    args.outputs.push_back(std::move(out));
  }

  // ---- executor ----
  std::unique_ptr<ExecutionRunner> runner = factory ? factory() : createHipExecutionRunner();
  if (!runner) return fail(summary, "executor_initialize", "no execution runner");
  if (Status st = runner->initialize(deviceId); !st.ok())
    return fail(summary, "executor_initialize", st.message);

  // ---- launch ----
  DynamicLibraryExecutionLaunch launch;
  launch.sharedLibraryPath = artifact->sharedLibraryPath;
  launch.symbolName = artifact->sharedLibrarySymbol;
  launch.regionProgram = artifact->regionProgram;
  if (Status st = runner->runDynamicLibraryArtifact(launch, args); !st.ok())
    return fail(summary, "kernel_launch", st.message);
  const double us = runner->lastKernelMicroseconds();
  if (us >= 0) summary.runtimeCounters["kernel_ns"] = (int64_t)(us * 1e3);
  summary.runtimeCounters["block_dim"] = inv.blockDim;
  summary.runtimeCounters["tiling_bytes"] = (int64_t)args.tiling.size();

  // ---- validate ----
  if (summary.validationRan) {
    auto cmp = compareRuntimeOutputs(args.outputs, expected, inv.atol, inv.rtol);
    if (!cmp) return fail(summary, "validate", cmp.error());
    summary.comparison = *cmp;
    summary.validationPassed = cmp->passed;
    if (!cmp->passed) return fail(summary, "validate", cmp->errorMessage);
  }

  // ---- write outputs ----
  for (size_t i = 0; i < inv.outputs.size(); ++i) {
    if (inv.outputs[i].path.empty()) continue;
    if (Status st = SaveNpy(inv.outputs[i].path, args.outputs[i]); !st.ok())
      return fail(summary, "write_outputs", st.message);
    summary.producedFiles.push_back(inv.outputs[i].path);
  }
  summary.success = true;
  return summary;
}

}  // namespace afirt
