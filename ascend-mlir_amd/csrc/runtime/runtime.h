// Host runtime behind the reference's runtime boundary, for the HIP backend:
// on-disk formats (npy, tiling bytes, artifact manifest, run manifest), the
// output comparator, the execution-runner seam and the single-task session
// that `runtime-session --run-manifest ... --run` drives.
//
// Reference interfaces mirrored here (paths relative to the reference tree):
//   include/Runtime/Support/Types.h:11-82            DType, NDArray, RunArgs
//   lib/Runtime/Support/NpyIO.cpp:17-164             LoadNpy / SaveNpy
//   lib/Runtime/Support/TilingSchema.cpp:13-100      TilingSchema::fromJson / pack
//   lib/Runtime/Support/TilingPack.cpp:43-89         packTilingBytes
//   lib/Runtime/Execution/OutputComparator.cpp:75-138 compareRuntimeOutputs
//   include/Runtime/Execution/ExecutionRunner.h:11-38 ExecutionRunner
//   lib/Runtime/Artifact/VecCubeArtifactBackend.cpp:62-106 out/manifest.txt
//   lib/Runtime/Artifact/RunManifest.cpp:175-290     run-manifest JSON
//   lib/Runtime/Execution/SimBackend.cpp:240-304,387-486 the run sequence
// The reference builds these on LLVMSupport; this library has no LLVM
// dependency, so errors travel as Expected<T> / Status carrying a message.
#pragma once

#include <cstddef>
#include <cstdint>
#include <map>
#include <memory>
#include <optional>
#include <string>
#include <utility>
#include <vector>

namespace afirt {

// ---------------------------------------------------------------- errors ----

struct Status {
  std::string message;  // empty = success
  bool ok() const { return message.empty(); }
  static Status success() { return {}; }
  static Status error(std::string m) { return Status{std::move(m)}; }
};

template <typename T>
class Expected {
 public:
  Expected(T value) : value_(std::move(value)) {}
  Expected(Status err) : error_(std::move(err.message)) {
    if (error_.empty()) error_ = "unknown error";
  }
  explicit operator bool() const { return value_.has_value(); }
  T &operator*() { return *value_; }
  const T &operator*() const { return *value_; }
  T *operator->() { return &*value_; }
  const T *operator->() const { return &*value_; }
  const std::string &error() const { return error_; }
  Status status() const { return value_ ? Status::success() : Status::error(error_); }

 private:
  std::optional<T> value_;
  std::string error_;
};

std::string format(const char *fmt, ...) __attribute__((format(printf, 1, 2)));

// ----------------------------------------------------------------- types ----

enum class DType { F16, BF16, F32, INT8, INT32, INT64 };
size_t dtypeBytes(DType d);
const char *dtypeName(DType d);                 // "f16", "bf16", ...
Expected<DType> parseDType(const std::string &name);

struct NDArray {
  std::vector<uint8_t> storage;  // owner (empty if external)
  void *data = nullptr;
  std::vector<int64_t> shape;
  DType dtype = DType::F16;

  void allocate() {
    storage.assign(nbytes(), 0);
    data = storage.data();
  }
  void setExternal(void *ptr) {
    storage.clear();
    data = ptr;
  }
  size_t numElements() const {
    size_t n = 1;  // empty shape = scalar
    for (auto s : shape) n *= static_cast<size_t>(s);
    return n;
  }
  size_t nbytes() const { return numElements() * dtypeBytes(dtype); }
};

struct RunArgs {
  std::vector<NDArray> inputs;
  std::vector<NDArray> outputs;   // pre-allocated, filled by the run
  std::vector<uint8_t> tiling;    // packed TilingData bytes (little-endian)
  // The caller's block_dim, in the reference's unit: a number of Ascend AI cores (its callers pass
  // 1, 8 or 40: python/runtime/executor.py:183, test/tools/runtime/test_capi_runtime.cpp:171-174,
  // examples/broadcast-add-reduce/run.sh:259).  It says nothing about a 256-CU GPU, so the HIP
  // runner records it and leaves the grid to the launcher, unless the process opts in with
  // AFIR_HIP_HONOUR_BLOCK_DIM=1 (then a positive block_dim is the number of workgroups).
  int block_dim = 1;
  // Workgroups to launch, for callers that mean a HIP grid (the run manifest's "hip_grid", the
  // tile search's block_dim_values); 0 = the launcher sizes the grid for the device.
  int hip_grid = 0;
  size_t workspace_size = 8192;
  // Extra timed launches of the same kernel on the same device buffers (the
  // kernels are pure functions of their inputs): the reported kernel time is the
  // fastest of 1 + timing_repeats launches.  For searches that score by time.
  int timing_repeats = 0;
  // > 1: the timed launches rotate over this many copies of the tensors on the device, so that
  // no launch finds its inputs in the last-level cache (256 MB on MI355X) because the launch
  // before it left them there.  The outputs handed back are those of the first copy.
  int buffer_sets = 1;
  // > 0 (with timing_repeats): before the timed launches the kernel is launched back to back for
  // this many milliseconds, and the timed launches then follow each other without a host
  // synchronisation in between; the reported time is their average.  The device needs 50-100 ms of
  // continuous work to settle at its sustained clocks; launches separated by synchronisations
  // never get there and read 3-10 % slow.
  double ramp_ms = 0.0;
};

// ------------------------------------------------------------------- npy ----

Expected<NDArray> LoadNpy(const std::string &path);
Status SaveNpy(const std::string &path, const NDArray &arr);

// ------------------------------------------------------------------ json ----

struct Json {
  enum Kind { Null, Bool, Number, String, Array, Object } kind = Null;
  bool boolean = false;
  double number = 0.0;
  bool is_integer = false;
  int64_t integer = 0;
  std::string string;
  std::vector<Json> array;
  std::vector<std::pair<std::string, Json>> object;  // insertion order kept

  const Json *get(const std::string &key) const;
  std::optional<std::string> getString(const std::string &key) const;
  std::optional<int64_t> getInteger(const std::string &key) const;
  std::optional<double> getNumber(const std::string &key) const;
  std::optional<bool> getBoolean(const std::string &key) const;
  const Json *getArray(const std::string &key) const;
  const Json *getObject(const std::string &key) const;
};
Expected<Json> parseJson(const std::string &text);
Expected<std::string> readTextFile(const std::string &path);

// ---------------------------------------------------------------- tiling ----

struct TilingField {
  std::string name;
  std::string type = "int64";  // "int64" (default) | "int32" | "int32_t"
};

class TilingSchema {
 public:
  static Expected<TilingSchema> fromJson(const std::string &path);
  static TilingSchema fromFields(std::vector<TilingField> fields);
  Expected<std::vector<uint8_t>> pack(
      const std::vector<std::pair<std::string, int64_t>> &params) const;
  const std::vector<TilingField> &fields() const { return fields_; }
  size_t size() const { return fields_.size(); }

 private:
  std::vector<TilingField> fields_;
};

struct TilingBinding {
  std::string schemaPath;
  std::string params;      // "K=V,K=V"
  std::string binaryPath;
};
Expected<std::vector<uint8_t>> packTilingBytes(const std::optional<TilingBinding> &tiling);

// ------------------------------------------------------------ comparator ----

struct OutputComparisonResult {
  bool passed = false;
  double maxAbsDiff = 0.0;
  double meanAbsDiff = 0.0;
  size_t mismatches = 0;
  std::string errorMessage;
};
// Structural mismatches (count, shape, dtype, size, null data) are errors.
Expected<OutputComparisonResult> compareRuntimeOutputs(const std::vector<NDArray> &actual,
                                                       const std::vector<NDArray> &expected,
                                                       double atol, double rtol);

// -------------------------------------------------------------- artifact ----

enum class KernelKind { Vec, Cube, Mix };
const char *kernelKindName(KernelKind k);
Expected<KernelKind> parseKernelKind(const std::string &name);

struct KernelArtifact {
  std::string kernelName;
  KernelKind kernelKind = KernelKind::Vec;
  std::string socVersion = "gfx950";
  std::string artifactRoot;
  std::string deviceBinaryPath;     // the artifact descriptor (<name>.hipk)
  std::string sharedLibraryPath;    // library exporting the launcher
  std::string sharedLibrarySymbol;  // launcher symbol
  std::string manifestPath;         // <root>/out/manifest.txt
  std::string regionProgram;        // fused_region artifacts: the program text
  std::string codeObjectPath;       // fused_region artifacts: kernels compiled for the program ("" = none)
  std::string codegenNote;          // why there is no code object, when there is none
  bool codeObjectPreferred = false; // the code object outranks a matching hand-tuned family
};

// The descriptor a "compiled" fused region consists of on this backend: the
// kernels are precompiled in the kernel library, so an artifact names one.
struct HipKernelDescriptor {
  std::string kernelName;   // name the caller launches by
  std::string hipKernel;    // family name in the kernel library's registry
  std::string library;      // path or soname of the kernel library ("" = default)
  std::string symbol;       // launcher symbol
  std::string program;      // hip_kernel == "fused_region": the region program text
  // Kernels compiled for the program (hipcc --genco of the emitted source):
  // file name beside the descriptor, and the directory it was written to.
  std::string codeObject;
  std::string codeObjectDir;
  bool codeObjectPreferred = false;   // compiled with explicit emit options: run it even where a hand-tuned family matches
};
// Path of the descriptor's code object: beside the descriptor when its
// directory is known and the file is there, else where it was compiled; ""
// when there is none.
std::string resolveCodeObject(const HipKernelDescriptor &d, const std::string &descriptorDir);
// Emits the HIP source of a region program to <dir>/<name>.hip and compiles it
// to <dir>/<name>.hsaco with hipcc ($HIPCC, PATH, /opt/rocm/bin).  Returns the
// code object's file name, or an error saying why there is none.
Expected<std::string> compileRegionCodeObject(const std::string &programText, const std::string &dir,
                                              const std::string &name,
                                              const std::map<std::string, int64_t> &emitOptions = {});
std::string serializeDescriptor(const HipKernelDescriptor &d);
Expected<HipKernelDescriptor> parseDescriptor(const std::string &text);

struct CompileRequest {
  std::string kernelSource;  // .mlir text naming the fused region, or a descriptor
  std::string outputDir;
  std::string kernelName;    // optional override
  std::string socVersion = "gfx950";
  std::optional<KernelKind> kernelKind;
  // Compile-time choices of the emitted region kernels: "tile_p", "tile_q",
  // "unroll" (csrc/target/hip_emitter.h: EmitOptions); absent = defaults.
  std::map<std::string, int64_t> emitOptions;
};
// Source -> artifact directory: <out>/<name>.hipk + <out>/out/manifest.txt.
Expected<KernelArtifact> compileArtifact(const CompileRequest &request);
Expected<KernelArtifact> loadArtifactFromRoot(const std::string &artifactRoot);
// What a kernel source compiles to: an explicit `hip_kernel=<family>` request
// or a function named after a family gives that family; MLIR text (linalg /
// AFIR) is translated to a fused-region program (csrc/target/mlir_translate.h).
Expected<HipKernelDescriptor> compileSourceText(const std::string &sourceText,
                                                const std::string &nameHint);

// Location of libafir_hip_kernels.so: $AFIR_HIP_KERNELS_LIB, else next to this
// library, else the bare soname for the dynamic loader to resolve.
std::string defaultKernelLibraryPath();

// ---------------------------------------------------------- run manifest ----

struct TensorBinding {
  std::string name;
  std::string path;
  std::vector<int64_t> shape;
  std::optional<DType> dtype;
  // source = "task_output": the tensor is output `upstreamOutput` of task
  // `upstreamTask` of the same manifest (lib/Runtime/Artifact/RunManifest.cpp:107-118)
  bool fromTaskOutput = false;
  std::string upstreamTask, upstreamOutput;
};

struct ExecutionInvocation {
  std::vector<TensorBinding> inputs, outputs, expectedOutputs;
  std::optional<TilingBinding> tiling;
  int blockDim = 1;
  int hipGrid = 0;        // "hip_grid": workgroups to launch, 0 = the launcher's choice
  size_t workspaceSize = 8192;
  bool enableProfiling = false;
  double atol = 1.0;
  double rtol = 1e-2;
};

struct RunTaskSpec {
  std::string taskId;
  std::string artifactRoot;
  std::vector<std::string> dependencies;
  ExecutionInvocation invocation;
};

struct RunManifestSpec {
  std::string backend;  // "hip" (also accepts the reference's "sim" / "npu")
  std::vector<RunTaskSpec> tasks;
};
Expected<RunManifestSpec> loadRunManifest(const std::string &path);

// ---------------------------------------------------------------- runner ----

enum class ExecutionRunnerMode { Simulation, RealDevice };

struct FileExecutionLaunch {
  std::string binaryPath;  // artifact descriptor
  std::string kernelName;
  uint32_t magic = 0;
};
struct DynamicLibraryExecutionLaunch {
  std::string sharedLibraryPath;
  std::string symbolName;
  // Non-empty: the artifact is a fused-region program.  It is registered with
  // the library (afir_hip_region_register) and launched by handle instead of
  // through a 16-slot launcher symbol.
  std::string regionProgram;
  // Optional code object compiled for that program; attached after
  // registration so the launch runs the compiled kernels.
  std::string codeObjectPath;
  bool preferCodeObject = false;
};

class ExecutionRunner {
 public:
  virtual ~ExecutionRunner() = default;
  virtual ExecutionRunnerMode mode() const = 0;
  virtual Status initialize(int deviceId = 0) = 0;
  virtual Status runFile(const FileExecutionLaunch &launch, RunArgs &args) = 0;
  virtual Status runDynamicLibraryArtifact(const DynamicLibraryExecutionLaunch &launch,
                                           RunArgs &args) = 0;
  // Kernel time of the last run in microseconds (HIP events), < 0 if unknown.
  virtual double lastKernelMicroseconds() const { return -1.0; }
  // Kernels the last run of a fused-region program went to: "family" (a hand-tuned
  // kernel), "compiled" (the artifact's code object) or "interpreter" (the library's
  // generic kernel, several times slower); "" for launcher-symbol artifacts.
  virtual std::string lastRegionRoute() const { return ""; }
  // The last kernel the last run launched and its grid; "" / 0 if unknown.  gridSource says who
  // chose the grid: "launcher", "hip_grid" or "block_dim" (AFIR_HIP_HONOUR_BLOCK_DIM=1).
  struct LaunchedGrid {
    std::string kernel, source;
    uint32_t workgroups = 0, threads = 0;
  };
  virtual LaunchedGrid lastLaunchedGrid() const { return {}; }
};

// The MI355X runner: alloc -> H2D -> launch -> sync -> D2H -> free
// (shape of lib/Runtime/Execution/NativeExecutionRunner.cpp:372-528,616-802).
std::unique_ptr<ExecutionRunner> createHipExecutionRunner();

constexpr uint32_t kMagicAIVec = 0x41415246u;
constexpr uint32_t kMagicAICube = 0x41494343u;

// --------------------------------------------------------------- session ----

using RunnerFactory = std::unique_ptr<ExecutionRunner> (*)();

struct SessionSummary {
  bool success = false;
  std::string backend = "hip";
  bool validationRan = false;
  bool validationPassed = false;
  std::string errorStage;     // artifact | bindings | executor_initialize |
                              // kernel_launch | validate | write_outputs
  std::string errorMessage;   // without the [hip:<stage>] prefix
  std::string rawErrorMessage;
  std::vector<std::string> producedFiles;
  std::map<std::string, std::string> runtimeAttributes;
  std::map<std::string, int64_t> runtimeCounters;
  OutputComparisonResult comparison;
  // Profiling (tasks with "profiling": true): one trace.json per task, schema
  // version 1 of lib/Runtime/Execution/SimBackend.cpp:314-374; score =
  // cycle_count = the kernel's duration in nanoseconds.
  struct ProfileArtifact {
    std::string taskId;
    std::string path;
    int64_t score = 0;
    int64_t cycleCount = 0;
  };
  std::string sessionId;
  std::vector<ProfileArtifact> profileArtifacts;
  std::string retainedSummaryPath;   // session_summary.json, when profiles were retained
};

// Runs one task: load artifact, bind inputs, allocate outputs from expected
// shapes, launch, validate, write outputs.
// profileDirectory: where a profiling task writes its trace.json ("" = nowhere).
SessionSummary runSingleTask(const RunTaskSpec &task, RunnerFactory factory, int deviceId,
                             const std::string &profileDirectory = "", const std::string &sessionId = "");

// Execution order of a manifest's tasks: Kahn's algorithm over `dependencies`,
// ready tasks in manifest order (lib/Runtime/Execution/TaskGraph.cpp:33-79).
// Errors: "empty task id", "duplicate task id", "unknown task dependency",
// "task graph contains a cycle".
Expected<std::vector<size_t>> planTasks(const RunManifestSpec &manifest);

// Serial session over all tasks in plan order.  An input bound to a task
// output reads the file that task wrote; outputs without a path are
// materialised as <workingDirectory>/<task>__<name>.npy
// (lib/Runtime/Execution/ExecutionSession.cpp:62-134,511-559).  Stops at the
// first failing task; the summary is the failing task's, or the merged one
// (validation passed = every validating task passed; counters carry a
// "<task>." prefix when there is more than one task).
// Profiling tasks write <workingDirectory>/opprof/hip/<task>/trace.json.
SessionSummary runSession(const RunManifestSpec &manifest, RunnerFactory factory, int deviceId,
                          const std::string &workingDirectory);

// Copies a session's profile artifacts to <root>/<session id>/tasks/<task>.json,
// writes <root>/<session id>/session_summary.json (schema version 1 of
// lib/Runtime/Profile/ProfileUtils.cpp:134-345: session_id, backend,
// task_count, successful_task_count, failed_task_count, tasks[{task_id,
// profile_path, score, cycle_count}], runtime{attributes, counters},
// total_score, total_cycle_count) and keeps the `keep` newest sessions under
// root.  Rewrites the summary's artifact paths to the retained copies.
Status retainProfileArtifacts(SessionSummary &summary, const std::string &root, size_t keep = 20);

}  // namespace afirt
