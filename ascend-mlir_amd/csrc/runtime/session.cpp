// Single-task session: the run sequence of the reference's backend
// (lib/Runtime/Execution/SimBackend.cpp:240-304,387-486) on the HIP runner:
// load artifact -> pack tiling -> load input .npy -> allocate outputs from the
// expected shapes -> launch -> compare -> save outputs.  Errors carry the
// stage they happened in, as "[hip:<stage>] message".
#include <deque>
#include <map>

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
  launch.codeObjectPath = artifact->codeObjectPath;
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

Expected<std::vector<size_t>> planTasks(const RunManifestSpec &manifest) {
  const auto &tasks = manifest.tasks;
  std::map<std::string, size_t> indexById;
  for (size_t i = 0; i < tasks.size(); ++i) {
    if (tasks[i].taskId.empty()) return Status::error("empty task id");
    if (!indexById.emplace(tasks[i].taskId, i).second) return Status::error("duplicate task id");
  }
  std::vector<size_t> indegree(tasks.size(), 0);
  std::vector<std::vector<size_t>> outgoing(tasks.size());
  for (size_t i = 0; i < tasks.size(); ++i)
    for (const std::string &dep : tasks[i].dependencies) {
      auto it = indexById.find(dep);
      if (it == indexById.end()) return Status::error("unknown task dependency");
      outgoing[it->second].push_back(i);
      ++indegree[i];
    }
  std::deque<size_t> ready;
  for (size_t i = 0; i < tasks.size(); ++i)
    if (indegree[i] == 0) ready.push_back(i);
  std::vector<size_t> order;
  while (!ready.empty()) {
    const size_t i = ready.front();
    ready.pop_front();
    order.push_back(i);
    for (size_t next : outgoing[i])
      if (--indegree[next] == 0) ready.push_back(next);
  }
  if (order.size() != tasks.size()) return Status::error("task graph contains a cycle");
  return order;
}

SessionSummary runSession(const RunManifestSpec &manifest, RunnerFactory factory, int deviceId,
                          const std::string &workingDirectory) {
  SessionSummary merged;
  auto order = planTasks(manifest);
  if (!order) return fail(merged, "driver", order.error());
  const bool many = manifest.tasks.size() > 1;
  std::map<std::string, TensorBinding> produced;   // "<task>::<output>" -> where it was written
  merged.validationPassed = true;
  for (size_t index : *order) {
    RunTaskSpec task = manifest.tasks[index];
    for (TensorBinding &b : task.invocation.inputs) {
      if (!b.fromTaskOutput) continue;
      const std::string key = b.upstreamTask + "::" + b.upstreamOutput;
      auto it = produced.find(key);
      if (it == produced.end())
        return fail(merged, "bindings", "task input binding cannot resolve upstream output " + key +
                                            " for task " + task.taskId);
      b.path = it->second.path;
      if (b.shape.empty()) b.shape = it->second.shape;
      if (!b.dtype) b.dtype = it->second.dtype;
      b.fromTaskOutput = false;
    }
    for (size_t i = 0; i < task.invocation.outputs.size(); ++i) {
      TensorBinding &b = task.invocation.outputs[i];
      if (b.name.empty()) b.name = "output" + std::to_string(i);
      if (b.path.empty()) {
        if (workingDirectory.empty())
          return fail(merged, "bindings", "output '" + b.name + "' of task " + task.taskId +
                                              " has no path and the session has no working directory");
        b.path = workingDirectory + "/" + task.taskId + "__" + b.name + ".npy";
      }
    }
    SessionSummary s = runSingleTask(task, factory, deviceId);
    if (!s.success) {
      if (many) s.errorMessage = "task " + task.taskId + ": " + s.errorMessage;
      if (many) s.rawErrorMessage = std::string("[hip:") + s.errorStage + "] " + s.errorMessage;
      return s;
    }
    for (const TensorBinding &b : task.invocation.outputs) produced[task.taskId + "::" + b.name] = b;
    merged.validationRan = merged.validationRan || s.validationRan;
    if (s.validationRan) {
      merged.validationPassed = merged.validationPassed && s.validationPassed;
      if (s.comparison.maxAbsDiff > merged.comparison.maxAbsDiff) merged.comparison = s.comparison;
    }
    const std::string prefix = many ? task.taskId + "." : "";
    for (const auto &kv : s.runtimeAttributes) merged.runtimeAttributes[prefix + kv.first] = kv.second;
    for (const auto &kv : s.runtimeCounters) merged.runtimeCounters[prefix + kv.first] = kv.second;
    merged.producedFiles.insert(merged.producedFiles.end(), s.producedFiles.begin(), s.producedFiles.end());
  }
  merged.success = true;
  if (!merged.validationRan) merged.validationPassed = false;
  return merged;
}

}  // namespace afirt
