#include "hiprtc_compile.h"

#include <dlfcn.h>

#include <mutex>

namespace afir_target {

const std::vector<std::string> &regionCompileOptions() {
  static const std::vector<std::string> options = {"--offload-arch=gfx950", "-O3", "-nogpuinc", "-ffp-contract=off",
                                                   "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"};
  return options;
}

namespace {

// The few entry points used, with the prototypes of hip/hiprtc.h (a result of 0 is success).
struct Hiprtc {
  typedef void *Program;
  int (*create)(Program *, const char *, const char *, int, const char *const *, const char *const *) = nullptr;
  int (*compile)(Program, int, const char *const *) = nullptr;
  int (*logSize)(Program, size_t *) = nullptr;
  int (*log)(Program, char *) = nullptr;
  int (*codeSize)(Program, size_t *) = nullptr;
  int (*code)(Program, char *) = nullptr;
  int (*destroy)(Program *) = nullptr;
  const char *(*errorString)(int) = nullptr;
  std::string why;   // not empty: the library is unusable
};

const Hiprtc &hiprtc() {
  static Hiprtc api;
  static std::once_flag once;
  std::call_once(once, [] {
    void *lib = nullptr;
    for (const char *name : {"libhiprtc.so", "libhiprtc.so.7", "/opt/rocm/lib/libhiprtc.so"})
      if ((lib = dlopen(name, RTLD_NOW | RTLD_LOCAL))) break;
    if (!lib) {
      api.why = "libhiprtc.so cannot be loaded (" + std::string(dlerror() ? dlerror() : "not found") + ")";
      return;
    }
    auto sym = [&](const char *name, auto *slot) {
      *slot = reinterpret_cast<std::remove_pointer_t<decltype(slot)>>(dlsym(lib, name));
      if (!*slot && api.why.empty()) api.why = std::string("libhiprtc.so lacks ") + name;
    };
    sym("hiprtcCreateProgram", &api.create);
    sym("hiprtcCompileProgram", &api.compile);
    sym("hiprtcGetProgramLogSize", &api.logSize);
    sym("hiprtcGetProgramLog", &api.log);
    sym("hiprtcGetCodeSize", &api.codeSize);
    sym("hiprtcGetCode", &api.code);
    sym("hiprtcDestroyProgram", &api.destroy);
    sym("hiprtcGetErrorString", &api.errorString);
  });
  return api;
}

}  // namespace

std::string compileWithHiprtc(const std::string &source, std::vector<char> *image) {
  const Hiprtc &rtc = hiprtc();
  if (!rtc.why.empty()) return rtc.why;
  Hiprtc::Program program = nullptr;
  int rc = rtc.create(&program, source.c_str(), "region.hip", 0, nullptr, nullptr);
  if (rc != 0) return std::string("hiprtcCreateProgram: ") + rtc.errorString(rc);
  std::vector<const char *> options;
  for (const std::string &o : regionCompileOptions()) options.push_back(o.c_str());
  rc = rtc.compile(program, (int)options.size(), options.data());
  std::string why;
  if (rc != 0) {
    size_t n = 0;
    std::string log;
    if (rtc.logSize(program, &n) == 0 && n > 1) {
      log.resize(n);
      if (rtc.log(program, &log[0]) != 0) log.clear();
    }
    if (log.size() > 1500) log = log.substr(log.size() - 1500);
    why = std::string("hiprtc rejected the region source (") + rtc.errorString(rc) + "):\n" + log;
  } else {
    size_t n = 0;
    if ((rc = rtc.codeSize(program, &n)) != 0 || n == 0) {
      why = std::string("hiprtcGetCodeSize: ") + rtc.errorString(rc);
    } else {
      image->resize(n);
      if ((rc = rtc.code(program, image->data())) != 0) why = std::string("hiprtcGetCode: ") + rtc.errorString(rc);
    }
  }
  (void)rtc.destroy(&program);
  return why;
}

}  // namespace afir_target
