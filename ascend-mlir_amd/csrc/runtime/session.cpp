// Single-task session: the run sequence of the reference's backend
// (lib/Runtime/Execution/SimBackend.cpp:240-304,387-486) on the HIP runner:
// load artifact -> pack tiling -> load input .npy -> allocate outputs from the
// expected shapes -> launch -> compare -> save outputs.  Errors carry the
// stage they happened in, as "[hip:<stage>] message".
#include <dirent.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <ctime>
#include <deque>
#include <fstream>
#include <map>
#include <sstream>

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

std::string jsonString(const std::string &text) {
  std::string o = "\"";
  for (char c : text) {
    switch (c) {
      case '"': o += "\\\""; break;
      case '\\': o += "\\\\"; break;
      case '\n': o += "\\n"; break;
      case '\r': o += "\\r"; break;
      case '\t': o += "\\t"; break;
      default: o += c;
    }
  }
  return o + "\"";
}

bool makeDirsFor(const std::string &dir) {
  std::string path;
  std::istringstream parts(dir);
  if (!dir.empty() && dir[0] == '/') path = "/";
  for (std::string part; std::getline(parts, part, '/');) {
    if (part.empty()) continue;
    path += part + "/";
    if (mkdir(path.c_str(), 0755) != 0 && errno != EEXIST) return false;
  }
  return true;
}

std::string tensorArrayJson(const std::vector<TensorBinding> &bindings, const std::vector<NDArray> &arrays) {
  std::string o = "[";
  for (size_t i = 0; i < arrays.size(); ++i) {
    o += i ? ", " : "";
    o += "{\"name\": " + jsonString(i < bindings.size() ? bindings[i].name : "") + ", \"shape\": [";
    for (size_t d = 0; d < arrays[i].shape.size(); ++d) o += (d ? ", " : "") + std::to_string(arrays[i].shape[d]);
    o += std::string("], \"dtype\": \"") + dtypeName(arrays[i].dtype) + "\"}";
  }
  return o + "]";
}

// trace.json of one task: the keys of the reference's simulator profile
// artifact (lib/Runtime/Execution/SimBackend.cpp:314-374), backend "hip".
Status writeProfileTrace(const std::string &dir, const std::string &sessionId, const RunTaskSpec &task,
                         const KernelArtifact &artifact, const RunArgs &args, int64_t kernelNs,
                         bool validationPassed, std::string *path) {
  if (!makeDirsFor(dir)) return Status::error("cannot create profile directory: " + dir);
  const ExecutionInvocation &inv = task.invocation;
  std::string tilingPath;
  if (inv.tiling) {
    tilingPath = dir + "/tiling.bin";
    std::ofstream f(tilingPath, std::ios::binary | std::ios::trunc);
    if (!f) return Status::error("cannot write tiling artifact: " + tilingPath);
    f.write(reinterpret_cast<const char *>(args.tiling.data()), (std::streamsize)args.tiling.size());
  }
  *path = dir + "/trace.json";
  std::ofstream f(*path, std::ios::trunc);
  if (!f) return Status::error("cannot write profile artifact: " + *path);
  f << "{\n";
  f << "  \"schema_version\": 1,\n";
  f << "  \"backend\": \"hip\",\n";
  f << "  \"session_id\": " << jsonString(sessionId) << ",\n";
  f << "  \"task_id\": " << jsonString(task.taskId) << ",\n";
  f << "  \"kernel_name\": " << jsonString(artifact.kernelName) << ",\n";
  f << "  \"kernel_kind\": \"" << kernelKindName(artifact.kernelKind) << "\",\n";
  f << "  \"soc_version\": " << jsonString(artifact.socVersion) << ",\n";
  f << "  \"block_dim\": " << inv.blockDim << ",\n";
  f << "  \"workspace_size\": " << (long long)args.workspace_size << ",\n";
  f << "  \"cycle_count\": " << (long long)kernelNs << ",\n";
  f << "  \"elapsed_us\": " << (long long)((kernelNs + 999) / 1000) << ",\n";
  f << "  \"score\": " << (long long)kernelNs << ",\n";
  f << "  \"score_unit\": \"ns\",\n";
  f << "  \"validation_passed\": " << (validationPassed ? "true" : "false") << ",\n";
  f << "  \"artifact_root\": " << jsonString(artifact.artifactRoot) << ",\n";
  f << "  \"inputs\": " << tensorArrayJson(inv.inputs, args.inputs) << ",\n";
  f << "  \"outputs\": " << tensorArrayJson(inv.outputs, args.outputs) << ",\n";
  f << "  \"tiling\": {\"present\": " << (inv.tiling ? "true" : "false") << ", \"binary_path\": "
    << jsonString(tilingPath) << ", \"bytes\": " << args.tiling.size() << "}\n";
  f << "}\n";
  f.flush();
  if (!f) return Status::error("failed to flush profile artifact: " + *path);
  return Status::success();
}

}  // namespace

SessionSummary runSingleTask(const RunTaskSpec &task, RunnerFactory factory, int deviceId,
                             const std::string &profileDirectory, const std::string &sessionId) {
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
  args.hip_grid = inv.hipGrid;
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

  // A region program takes its extents from TilingData (dim_arg<A>_<D> for
  // every dimension of every argument).  A task without a tiling binding --
  // the reference's hand-written static kernels have none,
  // examples/real-npu-multikernel/prepare.sh:74-176 -- gets them from the
  // tensors it binds.
  if (!inv.tiling && !artifact->regionProgram.empty()) {
    std::vector<int64_t> dims;
    for (const NDArray &a : args.inputs) dims.insert(dims.end(), a.shape.begin(), a.shape.end());
    for (const NDArray &a : args.outputs) dims.insert(dims.end(), a.shape.begin(), a.shape.end());
    args.tiling.resize(dims.size() * sizeof(int64_t));
    std::memcpy(args.tiling.data(), dims.data(), args.tiling.size());
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
  launch.preferCodeObject = artifact->codeObjectPreferred;
  if (Status st = runner->runDynamicLibraryArtifact(launch, args); !st.ok())
    return fail(summary, "kernel_launch", st.message);
  const double us = runner->lastKernelMicroseconds();
  if (us >= 0) summary.runtimeCounters["kernel_ns"] = (int64_t)(us * 1e3);
  // how a fused-region task was run; "interpreter" is the slow route (no code object in the artifact)
  if (const std::string route = runner->lastRegionRoute(); !route.empty())
    summary.runtimeAttributes["region_route"] = route;
  summary.runtimeCounters["block_dim"] = inv.blockDim;
  // the grid that ran (block_dim is the reference's AI-core count and does not size it)
  if (const auto grid = runner->lastLaunchedGrid(); grid.workgroups) {
    summary.runtimeAttributes["grid"] = std::to_string(grid.workgroups) + "x" + std::to_string(grid.threads);
    summary.runtimeAttributes["grid_source"] = grid.source;
    summary.runtimeAttributes["kernel"] = grid.kernel;
  }
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

  // ---- profiling ----
  summary.sessionId = sessionId;
  if (inv.enableProfiling && !profileDirectory.empty()) {
    SessionSummary::ProfileArtifact p;
    p.taskId = task.taskId;
    p.score = p.cycleCount = us >= 0 ? (int64_t)(us * 1e3) : 0;
    if (Status st = writeProfileTrace(profileDirectory, sessionId, task, *artifact, args, p.score,
                                      !summary.validationRan || summary.validationPassed, &p.path);
        !st.ok())
      return fail(summary, "profiling", st.message);
    summary.producedFiles.push_back(p.path);
    summary.profileArtifacts.push_back(p);
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
  {
    // session id in the shape of the reference's working directory names
    // (runtime-session-XXXXXX, lib/Runtime/Execution/ExecutionSession.cpp:148-157)
    static const char kAlphabet[] = "abcdefghijklmnopqrstuvwxyz0123456789";
    unsigned seed = (unsigned)std::time(nullptr) ^ ((unsigned)getpid() << 12);
    std::string id = "runtime-session-";
    for (int i = 0; i < 6; ++i) {
      seed = seed * 1664525u + 1013904223u;
      id += kAlphabet[(seed >> 16) % 36];
    }
    merged.sessionId = id;
  }
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
    const std::string profileDir =
        workingDirectory.empty() ? "" : workingDirectory + "/opprof/hip/" + task.taskId;
    SessionSummary s = runSingleTask(task, factory, deviceId, profileDir, merged.sessionId);
    s.sessionId = merged.sessionId;
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
    merged.profileArtifacts.insert(merged.profileArtifacts.end(), s.profileArtifacts.begin(),
                                   s.profileArtifacts.end());
  }
  merged.success = true;
  if (!merged.validationRan) merged.validationPassed = false;
  return merged;
}

Status retainProfileArtifacts(SessionSummary &summary, const std::string &root, size_t keep) {
  if (summary.profileArtifacts.empty()) return Status::success();
  const std::string sessionDir = root + "/" + summary.sessionId, taskDir = sessionDir + "/tasks";
  if (!makeDirsFor(taskDir)) return Status::error("cannot create retained profile directory: " + taskDir);
  int64_t totalScore = 0, totalCycles = 0;
  for (SessionSummary::ProfileArtifact &p : summary.profileArtifacts) {
    const std::string dst = taskDir + "/" + p.taskId + ".json";
    std::ifstream in(p.path, std::ios::binary);
    std::ofstream out(dst, std::ios::binary | std::ios::trunc);
    if (!in || !out) return Status::error("cannot retain profile artifact " + p.path + " -> " + dst);
    out << in.rdbuf();
    p.path = dst;
    totalScore += p.score;
    totalCycles += p.cycleCount;
  }
  const std::string summaryPath = sessionDir + "/session_summary.json";
  std::ofstream f(summaryPath, std::ios::trunc);
  if (!f) return Status::error("cannot write retained session summary: " + summaryPath);
  const size_t n = summary.profileArtifacts.size();
  f << "{\n  \"schema_version\": 1,\n  \"session_id\": " << jsonString(summary.sessionId)
    << ",\n  \"backend\": " << jsonString(summary.backend) << ",\n  \"task_count\": " << n
    << ",\n  \"successful_task_count\": " << n << ",\n  \"failed_task_count\": 0,\n  \"tasks\": [\n";
  for (size_t i = 0; i < n; ++i) {
    const SessionSummary::ProfileArtifact &p = summary.profileArtifacts[i];
    f << "    {\n      \"task_id\": " << jsonString(p.taskId) << ",\n      \"profile_path\": " << jsonString(p.path)
      << ",\n      \"score\": " << p.score << ",\n      \"cycle_count\": " << p.cycleCount << "\n    }"
      << (i + 1 != n ? "," : "") << "\n";
  }
  f << "  ],\n  \"runtime\": {\n    \"attributes\": {\n";
  for (auto it = summary.runtimeAttributes.begin(); it != summary.runtimeAttributes.end(); ++it)
    f << "      " << jsonString(it->first) << ": " << jsonString(it->second)
      << (std::next(it) != summary.runtimeAttributes.end() ? "," : "") << "\n";
  f << "    },\n    \"counters\": {\n";
  for (auto it = summary.runtimeCounters.begin(); it != summary.runtimeCounters.end(); ++it)
    f << "      " << jsonString(it->first) << ": " << it->second
      << (std::next(it) != summary.runtimeCounters.end() ? "," : "") << "\n";
  f << "    }\n  },\n  \"total_score\": " << totalScore << ",\n  \"total_cycle_count\": " << totalCycles << "\n}\n";
  f.flush();
  if (!f) return Status::error("cannot flush retained session summary: " + summaryPath);
  summary.retainedSummaryPath = summaryPath;

  // keep the newest sessions only
  std::vector<std::pair<time_t, std::string>> sessions;
  if (DIR *d = opendir(root.c_str())) {
    while (dirent *e = readdir(d)) {
      const std::string name = e->d_name;
      if (name == "." || name == "..") continue;
      struct stat st;
      if (stat((root + "/" + name).c_str(), &st) == 0 && S_ISDIR(st.st_mode)) sessions.push_back({st.st_mtime, name});
    }
    closedir(d);
  }
  std::sort(sessions.begin(), sessions.end());
  for (size_t i = 0; i + keep < sessions.size(); ++i) {
    if (sessions[i].second == summary.sessionId) continue;
    const std::string dir = root + "/" + sessions[i].second;
    if (DIR *d = opendir((dir + "/tasks").c_str())) {
      while (dirent *e = readdir(d))
        if (e->d_name[0] != '.') std::remove((dir + "/tasks/" + e->d_name).c_str());
      closedir(d);
    }
    rmdir((dir + "/tasks").c_str());
    std::remove((dir + "/session_summary.json").c_str());
    rmdir(dir.c_str());
  }
  return Status::success();
}

}  // namespace afirt
