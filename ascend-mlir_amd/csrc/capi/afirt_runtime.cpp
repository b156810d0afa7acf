// afirt_* C API over the HIP runtime (declarations and the reference
// interfaces they mirror: include/afirt_runtime.h).
#include "afirt_runtime.h"

#include <cstring>
#include <fstream>
#include <iterator>
#include <memory>
#include <string>
#include <vector>

#include "../runtime/runtime.h"

namespace {

struct CompilerHandle {
  std::string socVersion = "gfx950";
  std::string arch;
  int optLevel = 2;
};

struct ExecutorHandle {
  bool initialized = false;
  int deviceId = 0;
  std::unique_ptr<afirt::ExecutionRunner> runner;
};

void writeErr(char *buf, size_t len, const std::string &msg) {
  if (!buf || len == 0) return;
  std::strncpy(buf, msg.c_str(), len - 1);
  buf[len - 1] = '\0';
}

afirt::Status runDescriptor(ExecutorHandle *h, const std::string &descriptorText, const std::string &descriptorDir,
                            const char *function_name, int num_inputs, const void **input_ptrs,
                            const size_t *input_bytes, int num_outputs, void **output_ptrs,
                            const size_t *output_bytes, const uint8_t *tiling_data,
                            size_t tiling_len, int block_dim, uint32_t magic) {
  using afirt::Status;
  const std::string fn = function_name ? function_name : "";
  if (fn.empty()) return Status::error("function name is required");
  if (num_inputs < 0 || num_outputs <= 0) return Status::error("invalid input/output binding counts");
  if ((num_inputs > 0 && (!input_ptrs || !input_bytes)) || !output_ptrs || !output_bytes)
    return Status::error("input/output pointer arrays are required");
  if (magic != afirt::kMagicAIVec && magic != afirt::kMagicAICube)
    return Status::error(afirt::format("unsupported kernel magic: 0x%08x", magic));

  auto d = afirt::parseDescriptor(descriptorText);
  if (!d) return Status::error(d.error());
  if (fn != d->kernelName && fn != d->hipKernel)
    return Status::error("kernel '" + fn + "' is not in the artifact (it holds '" + d->kernelName + "')");

  // byte-typed views: the API carries sizes, not shapes; the runner checks
  // them against the tiling data
  afirt::RunArgs args;
  args.block_dim = block_dim;
  for (int i = 0; i < num_inputs; ++i) {
    afirt::NDArray a;
    a.dtype = afirt::DType::INT8;
    a.shape = {(int64_t)input_bytes[i]};
    a.setExternal(const_cast<void *>(input_ptrs[i]));
    args.inputs.push_back(std::move(a));
  }
  for (int i = 0; i < num_outputs; ++i) {
    afirt::NDArray a;
    a.dtype = afirt::DType::INT8;
    a.shape = {(int64_t)output_bytes[i]};
    a.setExternal(output_ptrs[i]);
    args.outputs.push_back(std::move(a));
  }
  if (tiling_data && tiling_len) args.tiling.assign(tiling_data, tiling_data + tiling_len);

  afirt::DynamicLibraryExecutionLaunch launch;
  launch.sharedLibraryPath = d->library.empty() ? afirt::defaultKernelLibraryPath() : d->library;
  launch.symbolName = d->symbol;
  launch.regionProgram = d->program;
  launch.codeObjectPath = afirt::resolveCodeObject(*d, descriptorDir);
  launch.preferCodeObject = d->codeObjectPreferred;
  return h->runner->runDynamicLibraryArtifact(launch, args);
}

}  // namespace

extern "C" {

AfirtCompiler afirt_compiler_create(const char *soc_version, const char *arch, int opt_level) {
  auto *h = new CompilerHandle();
  if (soc_version && *soc_version) h->socVersion = soc_version;
  if (arch && *arch) h->arch = arch;
  h->optLevel = opt_level;
  return reinterpret_cast<AfirtCompiler>(h);
}

void afirt_compiler_destroy(AfirtCompiler compiler) {
  delete reinterpret_cast<CompilerHandle *>(compiler);
}

int afirt_compiler_compile(AfirtCompiler compiler, const char *src_file, const char *output_dir,
                           const char *kernel_name, char *out_bin_path, size_t buf_len) {
  auto *h = reinterpret_cast<CompilerHandle *>(compiler);
  if (!h) {
    writeErr(out_bin_path, buf_len, "compiler handle is null");
    return 1;
  }
  afirt::CompileRequest req;
  req.kernelSource = src_file ? src_file : "";
  req.outputDir = output_dir ? output_dir : "";
  req.kernelName = kernel_name ? kernel_name : "";
  req.socVersion = h->socVersion;
  if (h->arch.find("cube") != std::string::npos) req.kernelKind = afirt::KernelKind::Cube;
  auto artifact = afirt::compileArtifact(req);
  if (!artifact) {
    writeErr(out_bin_path, buf_len, artifact.error());
    return 1;
  }
  writeErr(out_bin_path, buf_len, artifact->deviceBinaryPath);
  return 0;
}

AfirtExecutor afirt_executor_create(void) {
  return reinterpret_cast<AfirtExecutor>(new ExecutorHandle());
}

void afirt_executor_destroy(AfirtExecutor executor) {
  delete reinterpret_cast<ExecutorHandle *>(executor);
}

int afirt_executor_initialize(AfirtExecutor executor, int device_id, char *err_buf, size_t err_len) {
  auto *h = reinterpret_cast<ExecutorHandle *>(executor);
  if (!h) {
    writeErr(err_buf, err_len, "executor handle is null");
    return 1;
  }
  if (device_id < 0) {
    writeErr(err_buf, err_len, "device id must be non-negative");
    return 1;
  }
  if (!h->runner) h->runner = afirt::createHipExecutionRunner();
  afirt::Status st = h->runner->initialize(device_id);
  if (!st.ok()) {
    writeErr(err_buf, err_len, st.message);
    return 1;
  }
  h->deviceId = device_id;
  h->initialized = true;
  return 0;
}

int afirt_executor_run(AfirtExecutor executor, const uint8_t *binary_data, size_t binary_len,
                       const char *function_name, int num_inputs, const void **input_ptrs,
                       const size_t *input_bytes, int num_outputs, void **output_ptrs,
                       const size_t *output_bytes, const uint8_t *tiling_data, size_t tiling_len,
                       int block_dim, uint32_t magic, char *err_buf, size_t err_len) {
  auto *h = reinterpret_cast<ExecutorHandle *>(executor);
  if (!h || !h->initialized) {
    writeErr(err_buf, err_len, "executor has not been initialized");
    return 1;
  }
  if (!binary_data || binary_len == 0) {
    writeErr(err_buf, err_len, "binary data is required");
    return 1;
  }
  std::string text(reinterpret_cast<const char *>(binary_data), binary_len);
  afirt::Status st = runDescriptor(h, text, "", function_name, num_inputs, input_ptrs, input_bytes,
                                   num_outputs, output_ptrs, output_bytes, tiling_data, tiling_len,
                                   block_dim, magic);
  if (!st.ok()) {
    writeErr(err_buf, err_len, st.message);
    return 1;
  }
  return 0;
}

int afirt_executor_run_file(AfirtExecutor executor, const char *binary_path,
                            const char *function_name, int num_inputs, const void **input_ptrs,
                            const size_t *input_bytes, int num_outputs, void **output_ptrs,
                            const size_t *output_bytes, const uint8_t *tiling_data,
                            size_t tiling_len, int block_dim, uint32_t magic, char *err_buf,
                            size_t err_len) {
  auto *h = reinterpret_cast<ExecutorHandle *>(executor);
  if (!h || !h->initialized) {
    writeErr(err_buf, err_len, "executor has not been initialized");
    return 1;
  }
  if (!binary_path || !*binary_path) {
    writeErr(err_buf, err_len, "binary path is required");
    return 1;
  }
  std::ifstream f(binary_path, std::ios::binary);
  if (!f) {
    writeErr(err_buf, err_len, std::string("cannot open ") + binary_path);
    return 1;
  }
  std::string text((std::istreambuf_iterator<char>(f)), std::istreambuf_iterator<char>());
  const std::string path = binary_path;
  const size_t slash = path.find_last_of('/');
  afirt::Status st = runDescriptor(h, text, slash == std::string::npos ? "." : path.substr(0, slash), function_name, num_inputs, input_ptrs, input_bytes,
                                   num_outputs, output_ptrs, output_bytes, tiling_data, tiling_len,
                                   block_dim, magic);
  if (!st.ok()) {
    writeErr(err_buf, err_len, st.message);
    return 1;
  }
  return 0;
}

int afirt_executor_last_launch(AfirtExecutor executor, int64_t *kernel_ns, uint32_t *workgroups,
                               uint32_t *threads, char *kernel_name, size_t name_len) {
  auto *h = reinterpret_cast<ExecutorHandle *>(executor);
  if (!h || !h->initialized || !h->runner) return 1;
  const double us = h->runner->lastKernelMicroseconds();
  const auto grid = h->runner->lastLaunchedGrid();
  if (us < 0 || !grid.workgroups) return 1;
  if (kernel_ns) *kernel_ns = (int64_t)(us * 1e3);
  if (workgroups) *workgroups = grid.workgroups;
  if (threads) *threads = grid.threads;
  writeErr(kernel_name, name_len, grid.kernel);
  return 0;
}

}  // extern "C"
