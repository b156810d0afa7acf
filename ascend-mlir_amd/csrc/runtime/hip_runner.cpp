// The MI355X execution runner and the single-task session.
//
// Runner sequence (shape of the reference's NativeExecutionRunner::runWithHandle
// and ::runDynamicLibraryArtifact, lib/Runtime/Execution/NativeExecutionRunner.cpp:
// 372-528, 616-802): allocate inputs / outputs / workspace on the device, copy
// the inputs in, call the artifact's launcher symbol with
// [inputs..., outputs..., workspace, tiling] in sixteen pointer slots, wait for
// the stream, copy the outputs back, free.  The tiling pointer handed to the
// launcher is the host copy: HIP kernels take their arguments by value.
//
// What the reference's runner does afresh for every run and this one keeps for its lifetime
// (an executor that runs the same artifact again and again, the serving case): the kernel
// library stays open, a region program stays registered with its code object loaded (keyed by
// program text, code object file and its modification time), and device buffers go back to a
// small pool instead of to hipFree, which synchronises the device.  Measured through
// afirt_executor_run on a [640, 512] f16 row sum: 0.76 ms per run before (0.47 of it loading the
// code object again), 0.1x ms after.
//
// Before anything is launched the caller's byte counts are checked against the
// sizes the tiling implies (afir_hip_argument_bytes), because the C API above
// carries no shapes and a short buffer would otherwise be read past its end on
// the device.
#include <dlfcn.h>

#include <fstream>
#include <iterator>
#include <hip/hip_runtime.h>

#include <sys/stat.h>

#include <chrono>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>

#include "runtime.h"

namespace afirt {

namespace {

struct KernelInfoView {  // layout of AfirHipKernelInfo (include/afir_hip_kernels.h)
  const char *name;
  const char *symbol;
  int num_inputs;
  int num_outputs;
  int num_tiling_fields;
  const char *const *tiling_fields;
  const char *signature;
};

using LaunchFn16 = uint32_t (*)(uint32_t, void *, void *, void *, void *, void *, void *, void *,
                                void *, void *, void *, void *, void *, void *, void *, void *,
                                void *, void *);
using LastErrorFn = const char *(*)();
using KernelCountFn = int (*)();
using KernelInfoFn = const KernelInfoView *(*)(int);
using ArgBytesFn = uint32_t (*)(const char *, const void *, size_t, size_t *, int);
using RegionRegisterFn = uint32_t (*)(const char *, size_t, uint64_t *);
using RegionUnregisterFn = uint32_t (*)(uint64_t);
using RegionInfoFn = uint32_t (*)(uint64_t, int *, int *, int *);
using RegionBytesFn = uint32_t (*)(uint64_t, const void *, size_t, size_t *, int);
using RegionLaunchFn = uint32_t (*)(uint64_t, uint32_t, void *, int, void *const *, void *,
                                    const void *, size_t);

std::string hipErr(const char *what, hipError_t e) {
  return std::string(what) + " failed: " + hipGetErrorString(e);
}

class HipExecutionRunner final : public ExecutionRunner {
 public:
  ~HipExecutionRunner() override {
    dropRegions();
    for (auto &b : pool_) (void)hipFree(b.second);
    for (auto &l : libs_) dlclose(l.second);
    if (stream_) (void)hipStreamDestroy(stream_);
    if (ev0_) (void)hipEventDestroy(ev0_);
    if (ev1_) (void)hipEventDestroy(ev1_);
  }

  ExecutionRunnerMode mode() const override { return ExecutionRunnerMode::RealDevice; }

  Status initialize(int deviceId) override {
    if (deviceId < 0) return Status::error("device id must be non-negative");
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess) return Status::error(hipErr("hipGetDeviceCount", e));
    if (deviceId >= count)
      return Status::error(format("device %d is not present (%d HIP device(s) visible)", deviceId, count));
    e = hipSetDevice(deviceId);
    if (e != hipSuccess) return Status::error(hipErr("hipSetDevice", e));
    if (!stream_) {
      e = hipStreamCreate(&stream_);  // default priority
      if (e != hipSuccess) return Status::error(hipErr("hipStreamCreate", e));
      e = hipEventCreate(&ev0_);
      if (e == hipSuccess) e = hipEventCreate(&ev1_);
      if (e != hipSuccess) return Status::error(hipErr("hipEventCreate", e));
    }
    deviceId_ = deviceId;
    initialized_ = true;
    return Status::success();
  }

  Status runFile(const FileExecutionLaunch &launch, RunArgs &args) override {
    if (launch.magic != kMagicAIVec && launch.magic != kMagicAICube)
      return Status::error(format("unsupported kernel magic: 0x%08x", launch.magic));
    auto text = readTextFile(launch.binaryPath);
    if (!text) return Status::error("cannot open " + launch.binaryPath);
    auto d = parseDescriptor(*text);
    if (!d) return Status::error(d.error());
    DynamicLibraryExecutionLaunch dl;
    dl.sharedLibraryPath = d->library.empty() ? defaultKernelLibraryPath() : d->library;
    dl.symbolName = d->symbol;
    dl.regionProgram = d->program;
    const size_t slash = launch.binaryPath.find_last_of('/');
    dl.codeObjectPath = resolveCodeObject(*d, slash == std::string::npos ? "." : launch.binaryPath.substr(0, slash));
    dl.preferCodeObject = d->codeObjectPreferred;
    return runDynamicLibraryArtifact(dl, args);
  }

  Status runDynamicLibraryArtifact(const DynamicLibraryExecutionLaunch &launch,
                                   RunArgs &args) override {
    // one run at a time per runner: the stream, the timing events and what is kept between runs
    // are the runner's.  (The reference's C API has no locks and is called from one thread; threads
    // that share an executor here take turns.)
    std::lock_guard<std::mutex> runLock(runMutex_);
    lastKernelUs_ = -1.0;
    lastRegionRoute_.clear();
    lastGrid_ = {};
    if (!initialized_) return Status::error("execution runner has not been initialized");
    if (args.inputs.size() + args.outputs.size() + 2 > 16)
      return Status::error("too many tensor arguments for a launcher call (16 pointer slots)");

    void *lib = nullptr;
    if (auto it = libs_.find(launch.sharedLibraryPath); it != libs_.end()) {
      lib = it->second;
    } else {
      lib = dlopen(launch.sharedLibraryPath.c_str(), RTLD_NOW | RTLD_LOCAL);
      if (!lib)
        return Status::error("dlopen dynamic library artifact failed (" + launch.sharedLibraryPath +
                             "): " + dlerror());
      libs_[launch.sharedLibraryPath] = lib;   // open until the runner goes
    }

    auto lastError = reinterpret_cast<LastErrorFn>(dlsym(lib, "afir_hip_last_error"));
    LaunchFn16 launchFn = nullptr;
    RegionLaunchFn regionLaunch = nullptr;
    uint64_t region = 0;
    if (launch.regionProgram.empty()) {
      launchFn = reinterpret_cast<LaunchFn16>(dlsym(lib, launch.symbolName.c_str()));
      if (!launchFn) {
        const char *err = dlerror();
        return Status::error("dlsym " + launch.symbolName + " failed: " + (err ? err : "unknown"));
      }
      // ---- host-side validation against the shapes in the tiling bytes ----
      if (Status st = validate(lib, launch.symbolName, args); !st.ok()) return st;
    } else {
      // A region program stands where the reference has a device binary:
      // register it, check the buffers against the shapes, launch by handle.
      auto reg = reinterpret_cast<RegionRegisterFn>(dlsym(lib, "afir_hip_region_register"));
      auto unreg = reinterpret_cast<RegionUnregisterFn>(dlsym(lib, "afir_hip_region_unregister"));
      regionLaunch = reinterpret_cast<RegionLaunchFn>(dlsym(lib, "afir_hip_launch_region"));
      if (!reg || !unreg || !regionLaunch)
        return Status::error("library has no fused-region entry points (afir_hip_region_register)");
      auto why = [&]() { return std::string(lastError ? lastError() : ""); };
      // the same program with the same code object file (path, size, modification time) as an
      // earlier run: its registration, with the module already loaded
      std::string key = launch.sharedLibraryPath + '\n' + launch.codeObjectPath + '\n';
      if (!launch.codeObjectPath.empty()) {
        struct stat st {};
        if (stat(launch.codeObjectPath.c_str(), &st) != 0) return Status::error("cannot attach code object " + launch.codeObjectPath);
        key += format("%lld.%ld.%lld", (long long)st.st_mtim.tv_sec, (long)st.st_mtim.tv_nsec, (long long)st.st_size);
      }
      key += launch.preferCodeObject ? "\np\n" : "\n-\n";
      key += launch.regionProgram;
      if (auto it = regions_.find(key); it != regions_.end()) {
        region = it->second.handle;
      } else {
        if (regions_.size() >= kMaxCachedRegions) dropRegions();
        if (reg(launch.regionProgram.data(), launch.regionProgram.size(), &region) != 0)
          return Status::error("invalid region program in artifact: " + why());
        struct Undo {   // not kept unless everything below succeeds
          RegionUnregisterFn fn;
          uint64_t handle;
          ~Undo() { if (handle) fn(handle); }
        } undo{unreg, region};
        if (!launch.codeObjectPath.empty()) {
          // kernels compiled for this program run in place of the interpreter
          using AttachFn = uint32_t (*)(uint64_t, const void *, size_t);
          auto attach = reinterpret_cast<AttachFn>(dlsym(lib, "afir_hip_region_attach_code_object"));
          std::ifstream f(launch.codeObjectPath, std::ios::binary);
          if (!attach || !f) return Status::error("cannot attach code object " + launch.codeObjectPath);
          const std::string image((std::istreambuf_iterator<char>(f)), std::istreambuf_iterator<char>());
          if (attach(region, image.data(), image.size()) != 0)
            return Status::error("code object " + launch.codeObjectPath + " rejected: " + why());
          if (launch.preferCodeObject) {
            using PreferFn = uint32_t (*)(uint64_t, int);
            auto prefer = reinterpret_cast<PreferFn>(dlsym(lib, "afir_hip_region_prefer_code_object"));
            if (prefer) (void)prefer(region, 1);
          }
          // load it now: the first launch would otherwise do so between the timing events
          using LoadFn = uint32_t (*)(uint64_t);
          if (auto load = reinterpret_cast<LoadFn>(dlsym(lib, "afir_hip_region_load")))
            if (load(region) != 0) return Status::error("code object " + launch.codeObjectPath + " rejected: " + why());
        }
        undo.handle = 0;
        regions_[key] = CachedRegion{region, unreg};
      }
      if (Status st = validateRegion(lib, region, args, why); !st.ok()) return st;
      using RouteFn = const char *(*)(uint64_t, const void *, size_t);
      if (auto route = reinterpret_cast<RouteFn>(dlsym(lib, "afir_hip_region_route")))
        lastRegionRoute_ = route(region, args.tiling.data(), args.tiling.size());
    }

    // ---- device buffers ----
    std::vector<std::pair<size_t, void *>> allocs;
    // (every path that gets here has waited for the stream, or nothing was enqueued on the buffers)
    auto cleanup = [&]() {
      for (auto it = allocs.rbegin(); it != allocs.rend(); ++it) release(it->first, it->second);
      allocs.clear();
    };
    auto devAlloc = [&](size_t bytes, void **out) -> hipError_t {
      // an empty tensor still gets a valid, distinct pointer
      const size_t size = bytes ? bytes : 16;
      hipError_t e = acquire(size, out);
      if (e == hipSuccess) allocs.emplace_back(size, *out);
      return e;
    };

    void *slots[16] = {};
    size_t idx = 0;
    std::vector<void *> outDev;
    for (auto &in : args.inputs) {
      void *dev = nullptr;
      hipError_t e = devAlloc(in.nbytes(), &dev);
      if (e != hipSuccess) { cleanup(); return Status::error(hipErr("hipMalloc input", e)); }
      if (in.nbytes()) {
        e = hipMemcpyAsync(dev, in.data, in.nbytes(), hipMemcpyHostToDevice, stream_);
        if (e != hipSuccess) { cleanup(); return Status::error(hipErr("hipMemcpy input", e)); }
      }
      slots[idx++] = dev;
    }
    for (auto &out : args.outputs) {
      void *dev = nullptr;
      hipError_t e = devAlloc(out.nbytes(), &dev);
      if (e != hipSuccess) { cleanup(); return Status::error(hipErr("hipMalloc output", e)); }
      outDev.push_back(dev);
      slots[idx++] = dev;
    }
    void *workspace = nullptr;
    {
      const size_t ws = args.workspace_size < 16 ? 16 : args.workspace_size;
      hipError_t e = devAlloc(ws, &workspace);
      if (e != hipSuccess) { cleanup(); return Status::error(hipErr("hipMalloc workspace", e)); }
      e = hipMemsetAsync(workspace, 0, 16, stream_);  // error flag words start at zero
      if (e != hipSuccess) { cleanup(); return Status::error(hipErr("hipMemset workspace", e)); }
    }
    slots[idx++] = workspace;
    slots[idx++] = args.tiling.empty() ? nullptr : args.tiling.data();

    // further copies of the tensors for timed launches to rotate over
    const int nsets = args.buffer_sets > 1 && args.timing_repeats > 0 ? args.buffer_sets : 1;
    const size_t ntensors = args.inputs.size() + args.outputs.size();
    std::vector<std::vector<void *>> sets(nsets, std::vector<void *>(slots, slots + 16));
    for (int k = 1; k < nsets; ++k)
      for (size_t i = 0; i < ntensors; ++i) {
        const size_t bytes = i < args.inputs.size() ? args.inputs[i].nbytes() : args.outputs[i - args.inputs.size()].nbytes();
        void *dev = nullptr;
        hipError_t e = devAlloc(bytes, &dev);
        if (e == hipSuccess && i < args.inputs.size() && bytes)
          e = hipMemcpyAsync(dev, slots[i], bytes, hipMemcpyDeviceToDevice, stream_);
        if (e != hipSuccess) { cleanup(); return Status::error(hipErr("copy of the tensors for rotation", e)); }
        sets[k][i] = dev;
      }

    // ---- launch ----
    // The launcher's first argument is a number of workgroups (0 = its own choice).  The
    // caller's block_dim is an Ascend AI-core count and becomes that only on request.
    uint32_t bd = 0;
    lastGrid_.source = "launcher";
    if (args.hip_grid > 0) {
      bd = (uint32_t)args.hip_grid;
      lastGrid_.source = "hip_grid";
    } else if (const char *env = getenv("AFIR_HIP_HONOUR_BLOCK_DIM"); env && env[0] == '1' && args.block_dim > 0) {
      bd = (uint32_t)args.block_dim;
      lastGrid_.source = "block_dim";
    }
    double bestUs = -1.0;
    auto launchOnce = [&](void **use) -> uint32_t {
      if (regionLaunch) {
        const int nargs = (int)(args.inputs.size() + args.outputs.size());
        return regionLaunch(region, bd, stream_, nargs, use, workspace, args.tiling.data(), args.tiling.size());
      }
      return launchFn(bd, stream_, use[0], use[1], use[2], use[3], use[4], use[5], use[6], use[7], use[8],
                      use[9], use[10], use[11], use[12], use[13], use[14], use[15]);
    };
    auto launchFailed = [&](uint32_t rc) {
      std::string why = lastError ? lastError() : "";
      (void)hipStreamSynchronize(stream_);
      cleanup();
      return Status::error(format("dynamic library artifact launch failed: rc=%u", rc) +
                           (why.empty() ? "" : " (" + why + ")"));
    };
    const int repeats = args.timing_repeats > 0 ? args.timing_repeats : 0;
    const bool continuous = repeats > 0 && args.ramp_ms > 0;
    // the first launch (the only one without timing_repeats), and every launch when the timed
    // launches are separated by synchronisations
    for (int rep = 0; rep <= (continuous ? 0 : repeats); ++rep) {
      void **use = sets[rep % nsets].data();
      (void)hipEventRecord(ev0_, stream_);
      const uint32_t rc = launchOnce(use);
      if (rc != 0) return launchFailed(rc);
      (void)hipEventRecord(ev1_, stream_);
      hipError_t e = hipStreamSynchronize(stream_);
      if (e != hipSuccess) { cleanup(); return Status::error(hipErr("hipStreamSynchronize", e)); }
      float ms = 0.f;
      if (hipEventElapsedTime(&ms, ev0_, ev1_) == hipSuccess && (bestUs < 0 || (double)ms * 1e3 < bestUs))
        bestUs = (double)ms * 1e3;
    }
    if (continuous) {
      int next = 1;
      const auto until = std::chrono::steady_clock::now() + std::chrono::duration<double, std::milli>(args.ramp_ms);
      while (std::chrono::steady_clock::now() < until) {
        for (int i = 0; i < 16; ++i) {
          const uint32_t rc = launchOnce(sets[next++ % nsets].data());
          if (rc != 0) return launchFailed(rc);
        }
        (void)hipStreamSynchronize(stream_);
      }
      // the timed launches: one pair of events around all of them, the score is their average
      // (an event between every two launches costs about 2 us of idle device per launch)
      uint32_t rc = 0;
      (void)hipEventRecord(ev0_, stream_);
      for (int rep = 0; rep < repeats && rc == 0; ++rep) rc = launchOnce(sets[next++ % nsets].data());
      (void)hipEventRecord(ev1_, stream_);
      const hipError_t e = hipStreamSynchronize(stream_);
      if (rc != 0) return launchFailed(rc);
      if (e != hipSuccess) { cleanup(); return Status::error(hipErr("hipStreamSynchronize (timed launches)", e)); }
      float ms = 0.f;
      if (hipEventElapsedTime(&ms, ev0_, ev1_) == hipSuccess) bestUs = (double)ms * 1e3 / repeats;
    }
    lastKernelUs_ = bestUs;
    using LastLaunchFn = const char *(*)(uint32_t *, uint32_t *);
    if (auto last = reinterpret_cast<LastLaunchFn>(dlsym(lib, "afir_hip_last_launch")))
      if (const char *name = last(&lastGrid_.workgroups, &lastGrid_.threads)) lastGrid_.kernel = name;

    // ---- data errors reported through the workspace ----
    int32_t flag = 0;
    hipError_t e = hipMemcpy(&flag, workspace, sizeof flag, hipMemcpyDeviceToHost);
    if (e != hipSuccess) { cleanup(); return Status::error(hipErr("hipMemcpy workspace", e)); }
    if (flag != 0) {
      cleanup();
      return Status::error("kernel reported a data error: index out of range in gather");
    }

    for (size_t i = 0; i < args.outputs.size(); ++i) {
      if (!args.outputs[i].nbytes()) continue;
      e = hipMemcpy(args.outputs[i].data, outDev[i], args.outputs[i].nbytes(), hipMemcpyDeviceToHost);
      if (e != hipSuccess) { cleanup(); return Status::error(hipErr("hipMemcpy output", e)); }
    }
    cleanup();
    return Status::success();
  }

  double lastKernelMicroseconds() const override { return lastKernelUs_; }
  std::string lastRegionRoute() const override { return lastRegionRoute_; }
  LaunchedGrid lastLaunchedGrid() const override { return lastGrid_; }

 private:
  // ---- what is kept between runs ----
  struct CachedRegion {
    uint64_t handle;
    RegionUnregisterFn unregister;
  };
  static constexpr size_t kMaxCachedRegions = 64;
  static constexpr size_t kMaxPooledBytes = (size_t)4 << 30, kMaxPooledBuffers = 64;
  void dropRegions() {
    for (auto &r : regions_) (void)r.second.unregister(r.second.handle);
    regions_.clear();
  }
  // device buffers by exact size: a run of the same artifact asks for the same sizes again
  hipError_t acquire(size_t size, void **out) {
    auto it = pool_.find(size);
    if (it != pool_.end()) {
      *out = it->second;
      pool_.erase(it);
      pooledBytes_ -= size;
      return hipSuccess;
    }
    hipError_t e = hipMalloc(out, size);
    if (e != hipSuccess && !pool_.empty()) {   // give the pool back and try once more
      (void)hipGetLastError();
      for (auto &b : pool_) (void)hipFree(b.second);
      pool_.clear();
      pooledBytes_ = 0;
      e = hipMalloc(out, size);
    }
    return e;
  }
  void release(size_t size, void *p) {
    if (!p) return;
    if (pool_.size() < kMaxPooledBuffers && pooledBytes_ + size <= kMaxPooledBytes) {
      pool_.emplace(size, p);
      pooledBytes_ += size;
    } else {
      (void)hipFree(p);
    }
  }
  std::mutex runMutex_;
  std::map<std::string, void *> libs_;
  std::map<std::string, CachedRegion> regions_;
  std::multimap<size_t, void *> pool_;
  size_t pooledBytes_ = 0;

  Status validate(void *lib, const std::string &symbol, const RunArgs &args) {
    auto countFn = reinterpret_cast<KernelCountFn>(dlsym(lib, "afir_hip_kernel_count"));
    auto infoFn = reinterpret_cast<KernelInfoFn>(dlsym(lib, "afir_hip_kernel_info"));
    auto bytesFn = reinterpret_cast<ArgBytesFn>(dlsym(lib, "afir_hip_argument_bytes"));
    auto lastError = reinterpret_cast<LastErrorFn>(dlsym(lib, "afir_hip_last_error"));
    if (!countFn || !infoFn || !bytesFn)
      return Status::error("library exports no kernel registry (afir_hip_kernel_info): cannot "
                           "validate buffers for " + symbol);
    const KernelInfoView *info = nullptr;
    for (int i = 0; i < countFn(); ++i) {
      const KernelInfoView *k = infoFn(i);
      if (k && symbol == k->symbol) info = k;
    }
    if (!info) return Status::error("launcher symbol is not in the kernel registry: " + symbol);
    if ((int)args.inputs.size() != info->num_inputs)
      return Status::error(format("%s expects %d inputs, got %zu", info->name, info->num_inputs,
                                  args.inputs.size()));
    if ((int)args.outputs.size() != info->num_outputs)
      return Status::error(format("%s expects %d outputs, got %zu", info->name, info->num_outputs,
                                  args.outputs.size()));
    size_t want[16] = {};
    if (bytesFn(info->name, args.tiling.data(), args.tiling.size(), want, 16) != 0)
      return Status::error(std::string("invalid tiling data: ") + (lastError ? lastError() : ""));
    for (size_t i = 0; i < args.inputs.size(); ++i) {
      if (args.inputs[i].nbytes() != want[i])
        return Status::error(format("%s: input %zu holds %zu bytes, the tiling data implies %zu",
                                    info->name, i, args.inputs[i].nbytes(), want[i]));
      if (want[i] && !args.inputs[i].data)
        return Status::error(format("%s: input %zu has no data", info->name, i));
    }
    for (size_t i = 0; i < args.outputs.size(); ++i) {
      const size_t w = want[args.inputs.size() + i];
      if (args.outputs[i].nbytes() != w)
        return Status::error(format("%s: output %zu holds %zu bytes, the tiling data implies %zu",
                                    info->name, i, args.outputs[i].nbytes(), w));
      if (w && !args.outputs[i].data)
        return Status::error(format("%s: output %zu has no buffer", info->name, i));
    }
    return Status::success();
  }

  template <typename Why>
  Status validateRegion(void *lib, uint64_t region, const RunArgs &args, Why why) {
    auto infoFn = reinterpret_cast<RegionInfoFn>(dlsym(lib, "afir_hip_region_info"));
    auto bytesFn = reinterpret_cast<RegionBytesFn>(dlsym(lib, "afir_hip_region_argument_bytes"));
    if (!infoFn || !bytesFn) return Status::error("library cannot describe region programs");
    int nin = 0, nout = 0, nfields = 0;
    if (infoFn(region, &nin, &nout, &nfields) != 0) return Status::error(why());
    if ((int)args.inputs.size() != nin)
      return Status::error(format("region expects %d inputs, got %zu", nin, args.inputs.size()));
    if ((int)args.outputs.size() != nout)
      return Status::error(format("region expects %d outputs, got %zu", nout, args.outputs.size()));
    size_t want[16] = {};
    if (bytesFn(region, args.tiling.data(), args.tiling.size(), want, 16) != 0)
      return Status::error("invalid tiling data: " + why());
    for (size_t i = 0; i < args.inputs.size(); ++i) {
      if (args.inputs[i].nbytes() != want[i])
        return Status::error(format("region: input %zu holds %zu bytes, the tiling data implies %zu",
                                    i, args.inputs[i].nbytes(), want[i]));
      if (want[i] && !args.inputs[i].data) return Status::error(format("region: input %zu has no data", i));
    }
    for (size_t i = 0; i < args.outputs.size(); ++i) {
      const size_t w = want[args.inputs.size() + i];
      if (args.outputs[i].nbytes() != w)
        return Status::error(format("region: output %zu holds %zu bytes, the tiling data implies %zu",
                                    i, args.outputs[i].nbytes(), w));
      if (w && !args.outputs[i].data) return Status::error(format("region: output %zu has no buffer", i));
    }
    return Status::success();
  }

  bool initialized_ = false;
  int deviceId_ = 0;
  hipStream_t stream_ = nullptr;
  hipEvent_t ev0_ = nullptr, ev1_ = nullptr;
  double lastKernelUs_ = -1.0;
  std::string lastRegionRoute_;
  LaunchedGrid lastGrid_;
};

}  // namespace

std::unique_ptr<ExecutionRunner> createHipExecutionRunner() {
  return std::make_unique<HipExecutionRunner>();
}

}  // namespace afirt
