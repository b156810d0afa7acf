// C ABI of libafir_hip_kernels.so: launcher symbols in the reference's
// dynamic-library-artifact shape, a kernel registry and name-based dispatch.
// Declarations and the reference interfaces they stand in for are in
// include/afir_hip_kernels.h.
#include "afir_hip_kernels.h"

#include <cstddef>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>

#include <atomic>
#include <map>
#include <memory>
#include <mutex>
#include <vector>

#include <dlfcn.h>

#include <fstream>
#include <iterator>

#include "../kernels/kernels.h"
#include "family_programs.h"
#include "../kernels/region_launch.h"
#include "../target/hip_emitter.h"
#include "../target/hiprtc_compile.h"
#include "../target/region_program.h"

namespace {

thread_local std::string g_last_error;

uint32_t finish(const afir::LaunchStatus &st) {
  if (st.code == 0) {
    g_last_error.clear();
    return AFIR_HIP_OK;
  }
  g_last_error = st.message ? st.message : "unknown error";
  return st.code == 1 ? AFIR_HIP_E_INVALID : AFIR_HIP_E_LAUNCH;
}

uint32_t fail(uint32_t code, const std::string &msg) {
  g_last_error = msg;
  return code;
}

// TilingData fields are little-endian int64; gfx950 hosts are little-endian
// x86-64, so a memcpy is the decode.
bool read_fields(const void *tiling, int count, int64_t *dst) {
  if (!tiling) return false;
  std::memcpy(dst, tiling, sizeof(int64_t) * (size_t)count);
  return true;
}

const char *const kFieldsAddMul[] = {"dim_arg0_0", "dim_arg0_1"};
const char *const kFieldsRowsum[] = {"dim_arg0_0", "dim_arg0_1"};
const char *const kFieldsTranspose[] = {"dim_arg0_0", "dim_arg0_1", "dim_arg0_2"};
const char *const kFieldsGather[] = {"dim_arg0_0", "dim_arg0_1", "dim_arg1_0"};
const char *const kFieldsMatmul[] = {"dim_arg0_0", "dim_arg0_1", "dim_arg1_1", "alpha_f32_bits"};

const AfirHipKernelInfo kKernels[] = {
    {"fused_add_mul", "afir_hip_launch_fused_add_mul", 2, 1, 2, kFieldsAddMul,
     "(a f32[R,C], b f32[R,C]) -> out f32[R,C] = (a + b) * b"},
    {"broadcast_add_reducesum", "afir_hip_launch_broadcast_add_reducesum", 2, 1, 2, kFieldsRowsum,
     "(x f32[M,N], bias f32[N]) -> y f32[M] = sum_j (x[i,j] + bias[j])"},
    {"relu_broadcast_add_transpose", "afir_hip_launch_relu_broadcast_add_transpose", 2, 1, 3,
     kFieldsTranspose, "(x f16[B,M,N], c f16[N]) -> out f16[B,N,M] = relu(x[b,i,j]) + c[j]"},
    {"gather_scale_shift", "afir_hip_launch_gather_scale_shift", 4, 1, 3, kFieldsGather,
     "(table f16[V,D], indices i32[R], scale f16[D], shift f16[D]) -> out f16[R,D]"},
    {"matmul_add_leakyrelu", "afir_hip_launch_matmul_add_leakyrelu", 3, 1, 4, kFieldsMatmul,
     "(A bf16[M,K], B bf16[K,N], bias bf16[N]) -> out bf16[M,N] = leakyrelu(A@B + bias, alpha)"},
};
constexpr int kNumKernels = (int)(sizeof(kKernels) / sizeof(kKernels[0]));


// ---- registered region programs ----

// Programs that are exactly one of the hand-tuned kernels are routed to it
// (same arithmetic, faster data movement); everything else runs on the generic
// region kernel.  Matmul programs have no generic form: they must match.
enum class FastPath { None, AddMul, BcastAddRowsum, ReluBcastTranspose, GatherScaleShift, MatmulBiasLeaky, MatmulBiasLeakyF16 };

// A code object compiled for one program (afir_target::emitHipSource), loaded
// on first launch.
// Set when the process runs its static destructors: the HIP runtime may be gone by then.
bool g_process_exiting = false;

struct CompiledRegion {
  std::vector<char> image;
  std::mutex mutex;
  bool loaded = false;
  afir_target::EmitOptions options;   // read from the loaded module
  hipModule_t module = nullptr;
  std::map<std::string, hipFunction_t> functions;
  // the kernels that separate reads from writes: per segment whether it has one (filled at the
  // first launch), and per (kernel, dynamic LDS) how many of its workgroups fit a compute unit
  std::vector<afir_target::SpecPhased> phased;
  std::map<std::pair<std::string, unsigned>, int> resident;
  // The split / join row sum keeps its partial sums in one array of the code object.  Launches
  // of that form are chained through this event, so that one on another stream waits for the
  // join of the one before it instead of overwriting its partial sums.
  std::mutex split_mutex;
  hipEvent_t split_done = nullptr;
  hipStream_t split_stream = nullptr;
  bool split_recorded = false;
  ~CompiledRegion() {
    // at process exit the module and the event are left to the operating system: unloading
    // from a static destructor can run after the HIP runtime has shut down
    if (!loaded || g_process_exiting) return;
    (void)hipDeviceSynchronize();   // no launch of this module may still be running
    if (split_done) (void)hipEventDestroy(split_done);
    (void)hipModuleUnload(module);
  }
};

struct RegisteredRegion {
  afir_region::Program program;
  std::vector<std::string> fields;
  FastPath fast = FastPath::None;
  int fastArgs[4] = {-1, -1, -1, -1};  // argument index of each kernel operand
  float alpha = 0.f;
  bool relu = false;   // matmul epilogue ends in max(v, 0) instead of max(v, v * alpha)
  std::shared_ptr<CompiledRegion> compiled;   // null: the interpreter kernel runs the program
  bool preferCompiled = false;                // the attached code object outranks a hand-tuned family
};

// Loads the module if needed and looks a kernel up.  "" on success.
std::string compiled_function(CompiledRegion *c, const afir_region::Program &program, const std::string &name,
                              hipFunction_t *fn) {
  std::lock_guard<std::mutex> lock(c->mutex);
  if (!c->loaded) {
    hipModule_t m = nullptr;
    hipError_t e = hipModuleLoadData(&m, c->image.data());
    if (e != hipSuccess) {
      (void)hipGetLastError();
      return std::string("code object does not load: ") + hipGetErrorString(e);
    }
    hipDeviceptr_t sym = nullptr;
    size_t bytes = 0;
    unsigned long long hash = 0;
    e = hipModuleGetGlobal(&sym, &bytes, m, "afir_region_program_hash");
    if (e == hipSuccess && bytes == sizeof hash) e = hipMemcpyDtoH(&hash, sym, sizeof hash);
    if (e != hipSuccess || bytes != sizeof hash || hash != afir_target::programHash(program)) {
      (void)hipModuleUnload(m);
      (void)hipGetLastError();   // a symbol that is not there is reported here, not by a later launch
      return "code object was not built from this program";
    }
    int abi = -1;
    if (hipModuleGetGlobal(&sym, &bytes, m, "afir_region_emit_abi") != hipSuccess || bytes != sizeof abi ||
        hipMemcpyDtoH(&abi, sym, sizeof abi) != hipSuccess || abi != afir_target::kSpecAbiVersion) {
      (void)hipModuleUnload(m);
      (void)hipGetLastError();
      return "code object was emitted by another version of this library (its kernels and their arguments differ); "
             "compile the artifact again";
    }
    // the tile / unroll choices the kernels were emitted with (older objects: the defaults)
    int opts[3] = {0, 0, 0};
    if (hipModuleGetGlobal(&sym, &bytes, m, "afir_region_emit_options") == hipSuccess && bytes == sizeof opts &&
        hipMemcpyDtoH(opts, sym, sizeof opts) == hipSuccess) {
      c->options.tileP = opts[0];
      c->options.tileQ = opts[1];
      c->options.unroll = opts[2];
      if (!afir_target::checkEmitOptions(c->options).empty()) {
        (void)hipModuleUnload(m);
        return "code object carries unusable emit options";
      }
    } else {
      (void)hipGetLastError();
    }
    c->module = m;
    c->loaded = true;
  }
  if (name.empty()) return "";   // load only
  auto it = c->functions.find(name);
  if (it == c->functions.end()) {
    hipFunction_t f = nullptr;
    const hipError_t e = hipModuleGetFunction(&f, c->module, name.c_str());
    if (e != hipSuccess) {
      (void)hipGetLastError();
      return "code object lacks kernel " + name + ": " + hipGetErrorString(e);
    }
    it = c->functions.emplace(name, f).first;
  }
  *fn = it->second;
  return "";
}

bool is_push(const afir_region::Op &o, int rank, std::initializer_list<int> dims) {
  using afir_region::MapResult;
  if (o.code != afir_region::OpCode::Push || !o.slice.empty() || (int)o.map.size() != (int)dims.size()) return false;
  (void)rank;
  size_t i = 0;
  for (int d : dims) {
    if (o.map[i].kind != MapResult::IterDim || o.map[i].iterDim != d) return false;
    ++i;
  }
  return true;
}

// Recognises the five hand-tuned kernels among region programs.  Returns a
// diagnostic for matmul programs that match none.
std::string detect_fast_path(RegisteredRegion *r) {
  using afir_region::ElemType;
  using afir_region::MapResult;
  using afir_region::OpCode;
  const afir_region::Program &p = r->program;
  if (p.segments.size() != 1) return "";
  const afir_region::Segment &g = p.segments[0];
  if (g.outOffset.arg >= 0 || g.outOffset.constant != 0 || !g.outOffsetMore.empty()) return "";
  const std::vector<afir_region::Op> &ops = g.ops;
  auto type = [&](int a) { return p.args[a].type; };
  const ElemType out = p.output().type;
  const bool hasMatmul = !ops.empty() && ops[0].code == OpCode::Matmul;

  if (hasMatmul) {
    // [matmul A B, (push bias (d1), add)?, (leaky alpha | relu)?, store]: the epilogue kinds None, BiasAdd and
    // BiasAddLeakyRelu of lib/Conversion/MarkStructuredOps/AnnotateMixMatmulSemanticsPass.cpp:319-323, the
    // runtime's BiasAddRelu (include/Runtime/Mix/MatmulTilingTypes.h:13; the emitter tells Relu from LeakyRelu
    // by the vector ops, test/Target/cann-translate-mix-relu.mlir:22-23), and either activation without a bias
    size_t at = 1;
    int bias = -1;
    float alpha = 1.f;   // max(v, v * 1) is v
    // (the bias runs along the last iteration dim: d1, or d2 of a batched product)
    if (at + 1 < ops.size() && (g.rank == 3 ? is_push(ops[at], 3, {2}) : is_push(ops[at], 2, {1})) &&
        ops[at + 1].code == OpCode::Add) {
      bias = ops[at].arg;
      at += 2;
    }
    bool relu = false;
    if (at < ops.size() && ops[at].code == OpCode::Leaky) alpha = ops[at++].constant;
    else if (at < ops.size() && ops[at].code == OpCode::Relu) { relu = true; ++at; }
    if (at + 1 == ops.size() && ops[at].code == OpCode::Store) {
      const int a = ops[0].arg, b = ops[0].arg2;
      if (type(a) == ElemType::BF16 && type(b) == ElemType::BF16 && (bias < 0 || type(bias) == ElemType::BF16) &&
          out == ElemType::BF16) {
        r->fast = FastPath::MatmulBiasLeaky;
      } else if (type(a) == ElemType::F16 && type(b) == ElemType::F16 && (bias < 0 || type(bias) == ElemType::F32) &&
                 out == ElemType::F32) {
        r->fast = FastPath::MatmulBiasLeakyF16;
      } else {
        return "matmul regions are implemented for bf16 A, B, bias, out and for f16 A, B with f32 bias, out; "
               "this one has other types";
      }
      r->fastArgs[0] = a; r->fastArgs[1] = b; r->fastArgs[2] = bias;
      r->alpha = alpha;
      r->relu = relu;
      return "";
    }
    return "a matmul region must be matmul [-> bias add (per column)] [-> leaky relu | relu]; other epilogues are not implemented";
  }
  if (g.rank == 2 && ops.size() == 6 && out == ElemType::F32 && is_push(ops[0], 2, {0, 1}) &&
      is_push(ops[1], 2, {0, 1}) && ops[2].code == OpCode::Add && is_push(ops[3], 2, {0, 1}) &&
      ops[4].code == OpCode::Mul && type(ops[0].arg) == ElemType::F32 && type(ops[1].arg) == ElemType::F32 &&
      (ops[3].arg == ops[0].arg || ops[3].arg == ops[1].arg) && ops[0].arg != ops[1].arg) {
    // (x + y) * z with z one of x, y: out = (a + b) * b with b the repeated operand
    r->fast = FastPath::AddMul;
    r->fastArgs[1] = ops[3].arg;
    r->fastArgs[0] = ops[3].arg == ops[0].arg ? ops[1].arg : ops[0].arg;
    return "";
  }
  if (g.rank == 2 && ops.size() == 5 && out == ElemType::F32 && ops[2].code == OpCode::Add &&
      ops[3].code == OpCode::ReduceSum) {
    for (int swap = 0; swap < 2; ++swap) {
      const afir_region::Op &x = ops[swap], &b = ops[1 - swap];
      if (is_push(x, 2, {0, 1}) && is_push(b, 2, {1}) && type(x.arg) == ElemType::F32 &&
          type(b.arg) == ElemType::F32) {
        r->fast = FastPath::BcastAddRowsum;
        r->fastArgs[0] = x.arg; r->fastArgs[1] = b.arg;
        return "";
      }
    }
  }
  if (g.rank == 3 && ops.size() == 5 && out == ElemType::F16 && ops[3].code == OpCode::Add) {
    // out[b,j,i] = relu(x[b,i,j]) + c[j]: x through (d0,d2,d1), c through (d1)
    const afir_region::Op *x = nullptr, *c = nullptr;
    if (is_push(ops[0], 3, {0, 2, 1}) && ops[1].code == OpCode::Relu && is_push(ops[2], 3, {1})) { x = &ops[0]; c = &ops[2]; }
    if (is_push(ops[0], 3, {1}) && is_push(ops[1], 3, {0, 2, 1}) && ops[2].code == OpCode::Relu) { x = &ops[1]; c = &ops[0]; }
    if (x && type(x->arg) == ElemType::F16 && type(c->arg) == ElemType::F16) {
      r->fast = FastPath::ReluBcastTranspose;
      r->fastArgs[0] = x->arg; r->fastArgs[1] = c->arg;
      return "";
    }
  }
  if (g.rank == 2 && ops.size() == 6 && out == ElemType::F16 && ops[2].code == OpCode::Mul &&
      ops[4].code == OpCode::Add && is_push(ops[3], 2, {1})) {
    for (int swap = 0; swap < 2; ++swap) {
      const afir_region::Op &t = ops[swap], &sc = ops[1 - swap];
      if (t.code == OpCode::Push && t.slice.empty() && t.map.size() == 2 &&
          t.map[0].kind == MapResult::Gather && t.map[0].iterDim == 0 &&
          t.map[1].kind == MapResult::IterDim && t.map[1].iterDim == 1 && is_push(sc, 2, {1}) &&
          type(t.arg) == ElemType::F16 && type(sc.arg) == ElemType::F16 &&
          type(ops[3].arg) == ElemType::F16 && type(t.map[0].indexArg) == ElemType::I32) {
        r->fast = FastPath::GatherScaleShift;
        r->fastArgs[0] = t.arg; r->fastArgs[1] = t.map[0].indexArg;
        r->fastArgs[2] = sc.arg; r->fastArgs[3] = ops[3].arg;
        return "";
      }
    }
  }
  return "";
}

// The hand-tuned kernels take densely packed operands whose shapes are the
// iteration extents.  A program can match a family and still read only part of a
// tensor (a zero-offset extract_slice narrower than its operand keeps the plain
// 'push'), so the shapes of a launch decide: every routed operand must be walked
// with the strides of a dense tensor of exactly the extents the kernel assumes,
// from element 0.  Extents of 1 leave their stride free.
bool fast_path_fits(const RegisteredRegion &r, const afir_region::Resolved &res) {
  if (res.segments.size() != 1) return false;
  const afir_region::ResolvedSegment &seg = res.segments[0];
  const int64_t *sz = seg.size;
  auto dense = [&](const afir_region::ResolvedInput &in, std::initializer_list<int64_t> strides) {
    if (in.offset != 0 || in.gatherIterDim >= 0) return false;
    int k = 0;
    for (int64_t want : strides) {
      if (sz[k] > 1 && in.iterStride[k] != want) return false;
      ++k;
    }
    return true;
  };
  // the output is dense by construction: resolve() checks that the one segment covers it
  switch (r.fast) {
    case FastPath::None:
      return false;
    case FastPath::AddMul:
      for (const afir_region::ResolvedInput &in : seg.inputs)
        if (!dense(in, {sz[1], 1})) return false;
      return true;
    case FastPath::BcastAddRowsum:
      for (const afir_region::ResolvedInput &in : seg.inputs)
        if (!(in.arg == r.fastArgs[0] ? dense(in, {sz[1], 1}) : dense(in, {0, 1}))) return false;
      return true;
    case FastPath::ReluBcastTranspose:
      // iteration space (b, j, i); x is [b, i, j]
      for (const afir_region::ResolvedInput &in : seg.inputs)
        if (!(in.arg == r.fastArgs[0] ? dense(in, {sz[1] * sz[2], 1, sz[1]}) : dense(in, {0, 1, 0}))) return false;
      return true;
    case FastPath::GatherScaleShift:
      for (const afir_region::ResolvedInput &in : seg.inputs) {
        if (in.arg == r.fastArgs[0]) {
          // rows of exactly the iteration width, gathered along dim 0 from the whole table
          if (in.offset != 0 || in.gatherIterDim != 0 || (sz[1] > 1 && in.iterStride[1] != 1) ||
              in.gatherStride != sz[1] || in.gatherExtent != res.shapes[in.arg][0])
            return false;
        } else if (!dense(in, {0, 1})) {
          return false;
        }
      }
      return true;
    case FastPath::MatmulBiasLeaky:
    case FastPath::MatmulBiasLeakyF16:
      // resolve() has matched A and B (transposed, batched or not) against the segment; the bias is
      // read from element 0 along the last iteration dim
      for (const afir_region::ResolvedInput &in : seg.inputs)
        if (!(seg.rank == 3 ? dense(in, {0, 0, 1}) : dense(in, {0, 1}))) return false;
      return true;
  }
  return false;
}

std::mutex g_region_mutex;
std::map<uint64_t, std::shared_ptr<RegisteredRegion>> g_regions;
uint64_t g_next_region = 1;
// constructed after g_regions, so destroyed before it
struct ExitMarker {
  ~ExitMarker() { g_process_exiting = true; }
} g_exit_marker;

std::shared_ptr<RegisteredRegion> find_region(uint64_t handle) {
  std::lock_guard<std::mutex> lock(g_region_mutex);
  auto it = g_regions.find(handle);
  return it == g_regions.end() ? nullptr : it->second;
}

int region_type_code(afir_region::ElemType t) {
  switch (t) {
    case afir_region::ElemType::F16: return afir::kRegionF16;
    case afir_region::ElemType::BF16: return afir::kRegionBF16;
    case afir_region::ElemType::F32: return afir::kRegionF32;
    case afir_region::ElemType::I32: return afir::kRegionI32;
    case afir_region::ElemType::I64: return afir::kRegionI64;
    case afir_region::ElemType::I16: return afir::kRegionI16;
  }
  return afir::kRegionF32;
}

int region_op_code(afir_region::OpCode c, bool integer, bool narrow = false) {
  using afir_region::OpCode;
  if (integer && narrow) {
    switch (c) {
      case OpCode::Max: return afir::kRegionMaxI16;
      case OpCode::Min: return afir::kRegionMinI16;
      case OpCode::Relu: return afir::kRegionReluI16;
      default: break;
    }
  }
  if (integer) {
    switch (c) {
      case OpCode::Add: return afir::kRegionAddI;
      case OpCode::Sub: return afir::kRegionSubI;
      case OpCode::Mul: return afir::kRegionMulI;
      case OpCode::Max: return afir::kRegionMaxI;
      case OpCode::Min: return afir::kRegionMinI;
      case OpCode::Relu: return afir::kRegionReluI;
      case OpCode::Neg: return afir::kRegionNegI;
      default: break;   // push, const, dup as below; the rest does not occur (validate)
    }
  }
  switch (c) {
    case OpCode::Push: return afir::kRegionPush;
    case OpCode::Const: return afir::kRegionConst;
    case OpCode::Add: return afir::kRegionAdd;
    case OpCode::Sub: return afir::kRegionSub;
    case OpCode::Mul: return afir::kRegionMul;
    case OpCode::Div: return afir::kRegionDiv;
    case OpCode::Max: return afir::kRegionMax;
    case OpCode::Min: return afir::kRegionMin;
    case OpCode::Relu: return afir::kRegionRelu;
    case OpCode::Leaky: return afir::kRegionLeaky;
    case OpCode::Neg: return afir::kRegionNeg;
    case OpCode::Dup: return afir::kRegionDup;
    default: return -1;  // ReduceSum / Store are not interpreted per element
  }
}

std::string resolve_region(const RegisteredRegion &r, const void *tiling, size_t tiling_len,
                           afir_region::Resolved *out) {
  const size_t want = r.fields.size() * sizeof(int64_t);
  if ((!tiling && want) || tiling_len != want) {
    char buf[160];
    std::snprintf(buf, sizeof buf, "region: tiling data must be %zu bytes (%zu int64 fields), got %zu",
                  want, r.fields.size(), tiling_len);
    return buf;
  }
  std::vector<int64_t> dims(r.fields.size());
  if (want) std::memcpy(dims.data(), tiling, want);
  return afir_region::resolve(r.program, dims, out);
}

}  // namespace

namespace {
// (defined with the region registry below)
bool launch_family_region(int which, uint32_t block_dim, void *stream, std::initializer_list<void *> args,
                          void *workspace, std::initializer_list<int64_t> dims, uint32_t *rc);
}  // namespace

extern "C" {

const char *afir_hip_last_error(void) { return g_last_error.c_str(); }

const char *afir_hip_last_launch(uint32_t *workgroups, uint32_t *threads) {
  const afir::LaunchNote &note = afir::last_launch_note();
  if (workgroups) *workgroups = note.workgroups;
  if (threads) *threads = note.threads;
  return note.kernel;
}

uint32_t afir_hip_launch_fused_add_mul(uint32_t block_dim, void *stream, void *a, void *b,
                                       void *out, void * /*workspace*/, void *tiling) {
  int64_t f[2];
  if (!read_fields(tiling, 2, f)) return fail(AFIR_HIP_E_INVALID, "fused_add_mul: null tiling");
  return finish(afir::launch_fused_add_mul(static_cast<const float *>(a),
                                           static_cast<const float *>(b),
                                           static_cast<float *>(out), f[0], f[1], block_dim,
                                           static_cast<hipStream_t>(stream)));
}

uint32_t afir_hip_launch_broadcast_add_reducesum(uint32_t block_dim, void *stream, void *x,
                                                 void *bias, void *y, void * /*workspace*/,
                                                 void *tiling) {
  int64_t f[2];
  if (!read_fields(tiling, 2, f))
    return fail(AFIR_HIP_E_INVALID, "broadcast_add_reducesum: null tiling");
  {
    // The family's kernels give a wavefront or a workgroup to a row.  Rows of fewer than 512 chunks
    // (lanes shared between rows) and fewer than 1024 rows (a workgroup or several per row) measured
    // faster on the compiled region kernels: 100000 x 100 floats 2.5 -> 3.2 TB/s, 64 x 2^20 0.28 -> 5.4;
    // other shapes measured the same or slower there and stay here.
    const int64_t m = f[0], n = f[1], n4 = n / 4;
    const bool vec = n > 0 && n % 4 == 0 && ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(bias)) & 15u) == 0;
    uint32_t rc;
    if (m > 0 && x && bias && y && vec && (n4 < 512 || m < 1024) &&
        launch_family_region(0, block_dim, stream, {x, bias, y}, nullptr, {m, n, n, m}, &rc))
      return rc;
  }
  return finish(afir::launch_broadcast_add_reducesum(
      static_cast<const float *>(x), static_cast<const float *>(bias), static_cast<float *>(y),
      f[0], f[1], block_dim, static_cast<hipStream_t>(stream)));
}

uint32_t afir_hip_launch_relu_broadcast_add_transpose(uint32_t block_dim, void *stream, void *x,
                                                      void *c, void *out, void * /*workspace*/,
                                                      void *tiling) {
  int64_t f[3];
  if (!read_fields(tiling, 3, f))
    return fail(AFIR_HIP_E_INVALID, "relu_broadcast_add_transpose: null tiling");
  {
    // the specialised kernel takes whole 64 x 64 tiles of aligned tensors; other extents that are
    // multiples of 8 (every row on a 16-byte boundary) run on the compiled region kernels, tiles with
    // bounds checks and 128-bit accesses (64 x 1024 x 520: 2.3 -> 4.9 TB/s); the rest keeps the
    // family's 2-byte kernel, which measured faster than element accesses there
    const int64_t nb = f[0], m = f[1], n = f[2];
    const bool aligned = ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(c) |
                           reinterpret_cast<uintptr_t>(out)) & 15u) == 0;
    uint32_t rc;
    if (nb > 0 && m >= 64 && n >= 64 && x && c && out && aligned && m % 8 == 0 && n % 8 == 0 &&
        !(m % 64 == 0 && n % 64 == 0) &&
        launch_family_region(1, block_dim, stream, {x, c, out}, nullptr, {nb, m, n, n, nb, n, m}, &rc))
      return rc;
  }
  return finish(afir::launch_relu_broadcast_add_transpose(
      static_cast<const uint16_t *>(x), static_cast<const uint16_t *>(c),
      static_cast<uint16_t *>(out), f[0], f[1], f[2], block_dim,
      static_cast<hipStream_t>(stream)));
}

uint32_t afir_hip_launch_gather_scale_shift(uint32_t block_dim, void *stream, void *table,
                                            void *indices, void *scale, void *shift, void *out,
                                            void *workspace, void *tiling) {
  int64_t f[3];
  if (!read_fields(tiling, 3, f))
    return fail(AFIR_HIP_E_INVALID, "gather_scale_shift: null tiling");
  {
    // rows of fewer than 256 halves leave most lanes of the family's kernels idle; the compiled
    // region kernels give such rows one 16-byte chunk per lane (131072 x 64 table: 2.9 -> 6.6 TB/s).
    // Longer rows measured faster here.
    const int64_t rows = f[0], dim = f[1], nidx = f[2];
    const bool aligned = ((reinterpret_cast<uintptr_t>(table) | reinterpret_cast<uintptr_t>(scale) |
                           reinterpret_cast<uintptr_t>(shift) | reinterpret_cast<uintptr_t>(out)) & 15u) == 0;
    uint32_t rc;
    if (rows > 0 && nidx > 0 && table && indices && scale && shift && out && aligned && dim % 8 == 0 && dim > 0 &&
        dim < 256 &&
        launch_family_region(2, block_dim, stream, {table, indices, scale, shift, out}, workspace,
                             {rows, dim, nidx, dim, dim, nidx, dim}, &rc))
      return rc;
  }
  return finish(afir::launch_gather_scale_shift(
      static_cast<const uint16_t *>(table), static_cast<const int32_t *>(indices),
      static_cast<const uint16_t *>(scale), static_cast<const uint16_t *>(shift),
      static_cast<uint16_t *>(out), static_cast<int32_t *>(workspace), f[0], f[1], f[2],
      block_dim, static_cast<hipStream_t>(stream)));
}

uint32_t afir_hip_launch_matmul_add_leakyrelu(uint32_t block_dim, void *stream, void *a, void *b,
                                              void *bias, void *out, void * /*workspace*/,
                                              void *tiling) {
  int64_t f[4];
  if (!read_fields(tiling, 4, f))
    return fail(AFIR_HIP_E_INVALID, "matmul_add_leakyrelu: null tiling");
  if (!bias && f[0] != 0 && f[2] != 0)   // (the region route takes a null bias as "no bias")
    return fail(AFIR_HIP_E_INVALID, "matmul_add_leakyrelu: null tensor pointer");
  const uint32_t bits = (uint32_t)((uint64_t)f[3] & 0xffffffffu);
  float alpha;
  std::memcpy(&alpha, &bits, 4);
  return finish(afir::launch_matmul_add_leakyrelu(
      static_cast<const uint16_t *>(a), static_cast<const uint16_t *>(b),
      static_cast<const uint16_t *>(bias), static_cast<uint16_t *>(out), f[0], f[1], f[2], alpha,
      /*relu=*/false, block_dim, static_cast<hipStream_t>(stream)));
}

namespace {
uint32_t register_region(const char *program_text, size_t program_len, uint64_t *handle, bool generic);
}

uint32_t afir_hip_region_register(const char *program_text, size_t program_len, uint64_t *handle) {
  bool generic = false;
  if (const char *env = std::getenv("AFIR_HIP_REGION_GENERIC")) generic = *env && *env != '0';
  return register_region(program_text, program_len, handle, generic);
}

namespace {
uint32_t register_region(const char *program_text, size_t program_len, uint64_t *handle, bool generic) {
  if (!program_text || !handle) return fail(AFIR_HIP_E_INVALID, "region_register: null argument");
  auto r = std::make_shared<RegisteredRegion>();
  std::string why = afir_region::parse(std::string(program_text, program_len), &r->program);
  if (!why.empty()) return fail(AFIR_HIP_E_INVALID, why);
  r->fields = afir_region::tilingFieldNames(r->program);
  why = detect_fast_path(r.get());
  if (!why.empty()) return fail(AFIR_HIP_E_INVALID, why);
  if (generic && r->fast != FastPath::MatmulBiasLeaky && r->fast != FastPath::MatmulBiasLeakyF16)
    r->fast = FastPath::None;
  std::lock_guard<std::mutex> lock(g_region_mutex);
  *handle = g_next_region++;
  g_regions[*handle] = std::move(r);
  g_last_error.clear();
  return AFIR_HIP_OK;
}

// ---- the families' compiled form: lib/families/<family>.hsaco beside this library ----
struct FamilyRegion {
  const char *name;
  const char *program;
  std::once_flag once;
  uint64_t handle = 0;
  std::atomic<bool> usable{false};
};
FamilyRegion g_families[] = {
    {"broadcast_add_reducesum", afir_family::kBroadcastAddReducesum},
    {"relu_broadcast_add_transpose", afir_family::kReluBroadcastAddTranspose},
    {"gather_scale_shift", afir_family::kGatherScaleShift},
};

FamilyRegion *family_region(int which) {
  FamilyRegion &f = g_families[which];
  std::call_once(f.once, [&f] {
    if (const char *env = std::getenv("AFIR_HIP_FAMILY_FALLBACK"))
      if (*env == '0') return;
    Dl_info info;
    if (!dladdr(reinterpret_cast<const void *>(&afir_hip_kernel_count), &info) || !info.dli_fname) return;
    std::string dir(info.dli_fname);
    const size_t slash = dir.rfind('/');
    dir = slash == std::string::npos ? std::string(".") : dir.substr(0, slash);
    std::ifstream file(dir + "/families/" + f.name + ".hsaco", std::ios::binary);
    if (!file) return;
    const std::vector<char> image((std::istreambuf_iterator<char>(file)), std::istreambuf_iterator<char>());
    uint64_t h = 0;
    if (register_region(f.program, std::strlen(f.program), &h, /*generic=*/true) != AFIR_HIP_OK) return;
    if (afir_hip_region_attach_code_object(h, image.data(), image.size()) != AFIR_HIP_OK) {
      (void)afir_hip_region_unregister(h);
      return;
    }
    f.handle = h;
    f.usable = true;
  });
  return f.usable ? &f : nullptr;
}

// Runs a family's launch on its compiled region kernels.  False: not available (no code
// object was built, or it does not load); the caller goes on with the family's own kernels.
bool launch_family_region(int which, uint32_t block_dim, void *stream, std::initializer_list<void *> args,
                          void *workspace, std::initializer_list<int64_t> dims, uint32_t *rc) {
  FamilyRegion *f = family_region(which);
  if (!f) return false;
  std::vector<void *> a(args);
  std::vector<int64_t> t(dims);
  *rc = afir_hip_launch_region(f->handle, block_dim, stream, (int)a.size(), a.data(), workspace, t.data(),
                               t.size() * sizeof(int64_t));
  if (*rc == AFIR_HIP_E_LAUNCH) {   // e.g. a code object of another version: do without it from now on
    f->usable = false;
    g_last_error.clear();
    return false;
  }
  return true;
}
}  // namespace

uint32_t afir_hip_region_unregister(uint64_t handle) {
  std::lock_guard<std::mutex> lock(g_region_mutex);
  if (!g_regions.erase(handle)) return fail(AFIR_HIP_E_UNKNOWN, "no region program with that handle");
  return AFIR_HIP_OK;
}

uint32_t afir_hip_region_info(uint64_t handle, int *num_inputs, int *num_outputs,
                              int *num_tiling_fields) {
  auto r = find_region(handle);
  if (!r) return fail(AFIR_HIP_E_UNKNOWN, "no region program with that handle");
  if (num_inputs) *num_inputs = r->program.numInputs();
  if (num_outputs) *num_outputs = 1;
  if (num_tiling_fields) *num_tiling_fields = (int)r->fields.size();
  return AFIR_HIP_OK;
}

uint32_t afir_hip_region_prefer_code_object(uint64_t handle, int prefer) {
  auto r = find_region(handle);
  if (!r) return fail(AFIR_HIP_E_UNKNOWN, "no region program with that handle");
  std::lock_guard<std::mutex> lock(g_region_mutex);
  r->preferCompiled = prefer != 0;
  g_last_error.clear();
  return AFIR_HIP_OK;
}

const char *afir_hip_region_kernel(uint64_t handle) {
  auto r = find_region(handle);
  if (!r) return "";
  const bool matmul = r->fast == FastPath::MatmulBiasLeaky || r->fast == FastPath::MatmulBiasLeakyF16;
  if (r->preferCompiled && r->compiled && !matmul) return "fused_region_compiled";
  switch (r->fast) {
    case FastPath::AddMul: return "fused_add_mul";
    case FastPath::BcastAddRowsum: return "broadcast_add_reducesum";
    case FastPath::ReluBcastTranspose: return "relu_broadcast_add_transpose";
    case FastPath::GatherScaleShift: return "gather_scale_shift";
    case FastPath::MatmulBiasLeaky: return "matmul_add_leakyrelu";
    case FastPath::MatmulBiasLeakyF16: return "matmul_add_leakyrelu_f16";
    case FastPath::None: break;
  }
  return r->compiled ? "fused_region_compiled" : "fused_region";
}

uint32_t afir_hip_region_emit_source(uint64_t handle, char *buffer, size_t capacity, size_t *length) {
  auto r = find_region(handle);
  if (!r) return fail(AFIR_HIP_E_UNKNOWN, "no region program with that handle");
  if (!length) return fail(AFIR_HIP_E_INVALID, "region_emit_source: null length pointer");
  std::string source;
  const std::string why = afir_target::emitHipSource(r->program, "region", &source);
  if (!why.empty()) return fail(AFIR_HIP_E_INVALID, "no specialised kernel: " + why);
  *length = source.size();
  if (buffer && capacity) {
    const size_t n = source.size() < capacity - 1 ? source.size() : capacity - 1;
    std::memcpy(buffer, source.data(), n);
    buffer[n] = 0;
  }
  g_last_error.clear();
  return AFIR_HIP_OK;
}

uint32_t afir_hip_region_attach_code_object(uint64_t handle, const void *image, size_t image_len) {
  auto r = find_region(handle);
  if (!r) return fail(AFIR_HIP_E_UNKNOWN, "no region program with that handle");
  if (!image || image_len < 8) return fail(AFIR_HIP_E_INVALID, "region_attach_code_object: empty image");
  for (const afir_region::Segment &g : r->program.segments)
    if (!g.ops.empty() && g.ops[0].code == afir_region::OpCode::Matmul)
      return fail(AFIR_HIP_E_INVALID, "matmul regions run on the hand-written kernels and take no code object");
  auto c = std::make_shared<CompiledRegion>();
  c->image.assign(static_cast<const char *>(image), static_cast<const char *>(image) + image_len);
  std::lock_guard<std::mutex> lock(g_region_mutex);
  r->compiled = std::move(c);
  g_last_error.clear();
  return AFIR_HIP_OK;
}

uint32_t afir_hip_region_load(uint64_t handle) {
  auto r = find_region(handle);
  if (!r) return fail(AFIR_HIP_E_UNKNOWN, "no region program with that handle");
  std::shared_ptr<CompiledRegion> c;
  {
    std::lock_guard<std::mutex> lock(g_region_mutex);
    c = r->compiled;
  }
  if (!c) return AFIR_HIP_OK;   // nothing attached: the interpreter needs no loading
  const std::string why = compiled_function(c.get(), r->program, "", nullptr);
  if (!why.empty()) return fail(AFIR_HIP_E_LAUNCH, why);
  g_last_error.clear();
  return AFIR_HIP_OK;
}

uint32_t afir_hip_region_compile(uint64_t handle, void *image_out, size_t capacity, size_t *image_len) {
  auto r = find_region(handle);
  if (!r) return fail(AFIR_HIP_E_UNKNOWN, "no region program with that handle");
  std::string source;
  std::string why = afir_target::emitHipSource(r->program, "region", &source);
  if (!why.empty()) return fail(AFIR_HIP_E_INVALID, "no specialised kernel: " + why);
  std::vector<char> image;
  why = afir_target::compileWithHiprtc(source, &image);
  if (!why.empty()) return fail(AFIR_HIP_E_INVALID, why);
  if (image_len) *image_len = image.size();
  if (image_out && capacity >= image.size()) std::memcpy(image_out, image.data(), image.size());
  return afir_hip_region_attach_code_object(handle, image.data(), image.size());
}

const char *afir_hip_region_tiling_field(uint64_t handle, int index) {
  auto r = find_region(handle);
  if (!r || index < 0 || index >= (int)r->fields.size()) return "";
  return r->fields[index].c_str();  // owned by the registry entry
}

uint32_t afir_hip_region_argument_bytes(uint64_t handle, const void *tiling, size_t tiling_len,
                                        size_t *bytes, int max_args) {
  auto r = find_region(handle);
  if (!r) return fail(AFIR_HIP_E_UNKNOWN, "no region program with that handle");
  if (!bytes || max_args < (int)r->program.args.size())
    return fail(AFIR_HIP_E_INVALID, "region_argument_bytes: output array too small");
  afir_region::Resolved res;
  std::string why = resolve_region(*r, tiling, tiling_len, &res);
  if (!why.empty()) return fail(AFIR_HIP_E_INVALID, why);
  for (size_t i = 0; i < res.bytes.size(); ++i) bytes[i] = res.bytes[i];
  g_last_error.clear();
  return AFIR_HIP_OK;
}

const char *afir_hip_region_route(uint64_t handle, const void *tiling, size_t tiling_len) {
  auto r = find_region(handle);
  if (!r) {
    (void)fail(AFIR_HIP_E_UNKNOWN, "no region program with that handle");
    return "";
  }
  afir_region::Resolved res;
  const std::string why = resolve_region(*r, tiling, tiling_len, &res);
  if (!why.empty()) {
    (void)fail(AFIR_HIP_E_INVALID, why);
    return "";
  }
  g_last_error.clear();
  const bool is_matmul = r->fast == FastPath::MatmulBiasLeaky || r->fast == FastPath::MatmulBiasLeakyF16;
  bool has_code, prefer;
  {
    std::lock_guard<std::mutex> lock(g_region_mutex);
    has_code = r->compiled != nullptr;
    prefer = r->preferCompiled && has_code && !is_matmul;
  }
  if (r->fast != FastPath::None && !prefer && fast_path_fits(*r, res)) return "family";
  if (is_matmul) {
    (void)fail(AFIR_HIP_E_INVALID, "region: the matmul kernels read the bias from its first element, densely");
    return "";
  }
  if (const char *env = std::getenv("AFIR_HIP_REGION_INTERPRET"))
    if (*env && *env != '0') has_code = false;
  return has_code ? "compiled" : "interpreter";
}

uint32_t afir_hip_launch_region(uint64_t handle, uint32_t block_dim, void *stream, int num_args,
                                void *const *args, void *workspace, const void *tiling,
                                size_t tiling_len) {
  auto r = find_region(handle);
  if (!r) return fail(AFIR_HIP_E_UNKNOWN, "no region program with that handle");
  const int want = (int)r->program.args.size();
  if (num_args != want || !args) {
    char buf[128];
    std::snprintf(buf, sizeof buf, "region: expected %d tensor arguments, got %d", want, num_args);
    return fail(AFIR_HIP_E_INVALID, buf);
  }
  afir_region::Resolved res;
  std::string why = resolve_region(*r, tiling, tiling_len, &res);
  if (!why.empty()) return fail(AFIR_HIP_E_INVALID, why);
  for (int i = 0; i < want; ++i)
    if (res.bytes[i] && !args[i]) return fail(AFIR_HIP_E_INVALID, "region: null tensor pointer");

  bool prefer_compiled;
  {
    std::lock_guard<std::mutex> lock(g_region_mutex);
    prefer_compiled = r->preferCompiled && r->compiled != nullptr && r->fast != FastPath::MatmulBiasLeaky &&
                      r->fast != FastPath::MatmulBiasLeakyF16;
  }
  const bool is_matmul = r->fast == FastPath::MatmulBiasLeaky || r->fast == FastPath::MatmulBiasLeakyF16;
  const bool fits = r->fast != FastPath::None && fast_path_fits(*r, res);
  if (is_matmul && !fits)
    return fail(AFIR_HIP_E_INVALID, "region: the matmul kernels read the bias from its first element, densely");
  if (fits && !prefer_compiled) {
    const afir_region::ResolvedSegment &seg = res.segments[0];
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int *fa = r->fastArgs;
    void *out = args[want - 1];
    switch (r->fast) {
      case FastPath::AddMul:
        return finish(afir::launch_fused_add_mul(static_cast<const float *>(args[fa[0]]),
                                                 static_cast<const float *>(args[fa[1]]),
                                                 static_cast<float *>(out), seg.size[0], seg.size[1],
                                                 block_dim, st));
      case FastPath::BcastAddRowsum:
        return finish(afir::launch_broadcast_add_reducesum(
            static_cast<const float *>(args[fa[0]]), static_cast<const float *>(args[fa[1]]),
            static_cast<float *>(out), seg.size[0], seg.size[1], block_dim, st));
      case FastPath::ReluBcastTranspose:
        // iteration space (b, j, i) = output; x is [b, i, j]
        return finish(afir::launch_relu_broadcast_add_transpose(
            static_cast<const uint16_t *>(args[fa[0]]), static_cast<const uint16_t *>(args[fa[1]]),
            static_cast<uint16_t *>(out), seg.size[0], seg.size[2], seg.size[1], block_dim, st));
      case FastPath::GatherScaleShift:
        return finish(afir::launch_gather_scale_shift(
            static_cast<const uint16_t *>(args[fa[0]]), static_cast<const int32_t *>(args[fa[1]]),
            static_cast<const uint16_t *>(args[fa[2]]), static_cast<const uint16_t *>(args[fa[3]]),
            static_cast<uint16_t *>(out), static_cast<int32_t *>(workspace), res.shapes[fa[0]][0],
            seg.size[1], seg.size[0], block_dim, st));
      case FastPath::MatmulBiasLeaky:
      case FastPath::MatmulBiasLeakyF16: {
        // plain [M,K] x [K,N] products go to the direct-to-LDS / register-staged kernels, transposed
        // and batched operands to the layout kernels (launch_matmul_layouts picks)
        const afir_region::ResolvedOp &mm = seg.ops[0];
        const int b0 = seg.rank == 3 ? 1 : 0;
        return finish(afir::launch_matmul_layouts(
            static_cast<const uint16_t *>(args[fa[0]]), static_cast<const uint16_t *>(args[fa[1]]),
            fa[2] >= 0 ? args[fa[2]] : nullptr, out, r->fast == FastPath::MatmulBiasLeakyF16, mm.batch, seg.size[b0],
            mm.k, seg.size[b0 + 1], mm.transA, mm.transB, r->alpha, r->relu, block_dim, st));
      }
      case FastPath::None: break;
    }
  }

  auto aligned = [](const void *p, int64_t bytes) {
    return ((reinterpret_cast<uintptr_t>(p) + (uintptr_t)bytes) & 15u) == 0;
  };
  std::shared_ptr<CompiledRegion> compiled;
  {
    std::lock_guard<std::mutex> lock(g_region_mutex);
    compiled = r->compiled;
  }
  // AFIR_HIP_REGION_INTERPRET=1 keeps programs with a code object on the
  // interpreter kernel (the tests compare the two)
  if (const char *env = std::getenv("AFIR_HIP_REGION_INTERPRET"))
    if (*env && *env != '0') compiled.reset();
  afir_target::EmitOptions emit;
  if (compiled) {
    // load the module now: the grids below depend on the options it was emitted with
    hipFunction_t none = nullptr;
    const std::string no = compiled_function(compiled.get(), r->program, "", &none);
    if (!no.empty()) return fail(AFIR_HIP_E_LAUNCH, no);
    emit = compiled->options;
  }
  struct PendingSegment {
    int segment;
    afir_target::SpecArgs args;
    bool idx32;
    int mode;    // afir_target::SpecMode
    int rows;    // 1: the workgroup-per-row kernel of a reduce segment, 2: its form for few, long rows,
                 // 3: split (args.column_blocks workgroups per row) and join, for a handful of rows
    bool slim;   // the kernel whose lanes take one group each (short rows)
    bool elem;   // the kernel whose groups are single elements (rows off 16-byte boundaries)
    unsigned lds = 0;   // > 0: the kernel that stages a gathered operand's source row, with this much LDS
    bool stage_wave = false;   // ... its form with a wavefront per row
    bool phased = false;       // the kernel that separates reads from writes (lds: its row vectors)
    int64_t phased_bytes = 0;  // ... and what this launch of it reads
    int phased_rate = 0;       // ... at this many GB/s, by what it reads
  };
  // Hold of the emitted kernels that separate reads from writes: base + bytes read / rate.  The
  // rate the chip serves a launch's reads at depends on what is read (searched on [4096, 4096] f32
  // (a + b) * b, the split / relu / broadcast graph at [8192, 4096] f16 and 32768 gathered rows of
  // 1024 halves; 5 % either side costs about 1 %): two streamed operands 6700 GB/s, one 6900,
  // rows gathered through an index tensor 6100.  AFIR_REGION_PHASE_GBS overrides all three.
  const int region_hold_base_ns = afir::env_int("AFIR_REGION_PHASE_BASE_NS", 300, 0, 100000);
  const int region_hold_gbs = afir::env_int("AFIR_REGION_PHASE_GBS", 0, 100, 100000);
  auto region_hold_rate = [&](bool gathered, int streamed) {
    return region_hold_gbs ? region_hold_gbs : gathered ? 6100 : streamed > 1 ? 6700 : 6900;
  };
  // workgroups of a compiled kernel that fit a compute unit with `lds` bytes of dynamic LDS
  auto resident_per_cu = [&](const std::string &name, unsigned lds) -> int {
    hipFunction_t fn = nullptr;
    if (!compiled_function(compiled.get(), r->program, name, &fn).empty()) return 0;
    std::lock_guard<std::mutex> lock(compiled->mutex);
    const auto key = std::make_pair(name, lds);
    auto it = compiled->resident.find(key);
    if (it != compiled->resident.end()) return it->second;
    int n = 0;
    if (hipModuleOccupancyMaxActiveBlocksPerMultiprocessor(&n, fn, 256, lds) != hipSuccess) {
      (void)hipGetLastError();
      n = 0;
    }
    compiled->resident[key] = n;
    return n;
  };
  std::vector<PendingSegment> pending;   // compiled kernels to launch, non-empty segments only
  for (const afir_region::ResolvedSegment &seg : res.segments) {
    afir::RegionArgs a;
    std::memset(&a, 0, sizeof a);
    a.rank = seg.rank;
    for (int k = 0; k < 3; ++k) a.size[k] = k < seg.rank ? seg.size[k] : 1;
    a.reduce = seg.reduce ? 1 : 0;
    a.out_type = region_type_code(seg.outType);
    const int64_t oes = (int64_t)afir_region::elemTypeBytes(seg.outType);
    a.out = static_cast<char *>(args[want - 1]) + seg.outOffsetElems * oes;
    a.error_flag = static_cast<int32_t *>(workspace);
    const int last = seg.rank - 1;
    int64_t rows = 1;
    for (int k = 0; k < last; ++k) rows *= seg.size[k];
    a.out_vec = !seg.reduce && aligned(a.out, 0) && (rows <= 1 || (seg.size[last] * oes) % 16 == 0);
    a.ninputs = (int)seg.inputs.size();
    for (int i = 0; i < a.ninputs; ++i) {
      const afir_region::ResolvedInput &in = seg.inputs[i];
      afir::RegionInput &d = a.in[i];
      const int64_t es = (int64_t)afir_region::elemTypeBytes(in.type);
      d.base = args[in.arg];
      d.type = region_type_code(in.type);
      for (int k = 0; k < 3; ++k) d.stride[k] = in.iterStride[k];
      d.offset = in.offset;
      d.gdim = in.gatherIterDim;
      d.index = in.gatherIterDim >= 0 ? args[in.gatherIndexArg] : nullptr;
      d.gtype = region_type_code(in.gatherIndexType);
      d.gstride = in.gatherStride;
      d.gextent = in.gatherExtent;
      bool vec = aligned(d.base, in.offset * es);
      for (int k = 0; k < last; ++k)
        if (seg.size[k] > 1 && (in.iterStride[k] * es) % 16 != 0) vec = false;
      d.vec = vec ? 1 : 0;
      d.gvec = (in.gatherStride * es) % 16 == 0 ? 1 : 0;
    }
    a.nops = 0;
    for (const afir_region::ResolvedOp &op : seg.ops) {
      const bool integer = afir_region::isRegionInt(seg.outType);
      int code = region_op_code(op.code, integer, seg.outType == afir_region::ElemType::I16);
      if (op.code == afir_region::OpCode::Cast)   // a cast to f32 changes nothing
        code = op.castType == afir_region::ElemType::F16 ? (int)afir::kRegionCastF16
               : op.castType == afir_region::ElemType::BF16 ? (int)afir::kRegionCastBF16 : -1;
      if (code < 0) continue;
      afir::RegionOp &d = a.ops[a.nops++];
      d.code = code;
      d.input = op.input;
      d.constant = op.constant;
      if (integer && op.code == afir_region::OpCode::Const) {   // the integer, bit for bit
        const int32_t iv = (int32_t)op.constant;
        std::memcpy(&d.constant, &iv, sizeof iv);
      }
      d.depth = op.depth;
    }
    a.ntail = 0;
    for (const afir_region::ResolvedSegment::TailStep &t : seg.tail) {
      if (t.code == afir_region::OpCode::Cast && t.castType == afir_region::ElemType::F32) continue;
      afir::RegionOp &d = a.tail[a.ntail++];   // at most kMaxTailOps = kRegionMaxTail (validate)
      d.code = t.code == afir_region::OpCode::Cast
                   ? (t.castType == afir_region::ElemType::F16 ? (int)afir::kRegionCastF16 : (int)afir::kRegionCastBF16)
                   : region_op_code(t.code, false);
      d.constant = t.constant;
      d.depth = t.reversed ? 1 : 0;
    }
    if (compiled) {
      const int segment = (int)(&seg - res.segments.data());
      const afir_target::SpecShape shape = afir_target::specShape(r->program, segment, emit);
      const afir_target::SpecTile tile = afir_target::specTile(r->program, segment);
      const int wideW = shape.width;
      // Rows of fewer than 8 x unroll groups leave most of a lane's groups empty and make a wavefront's
      // loads touch short pieces of many rows: those run on the kernel whose lanes take one group each
      // (it exists with 32-bit positions, for launches whose 128-bit accesses are all aligned).
      const int64_t row_groups_all = (seg.size[seg.rank - 1] + wideW - 1) / wideW;
      bool skip = false;
      uint32_t failed = AFIR_HIP_OK;
      bool unaligned = false;   // set by a pass: some tensor's rows are off 16-byte boundaries
      // kind 0: the ordinary kernels; 1: one group per lane; 2: single-element groups
      auto prepare = [&](const afir::RegionArgs &ra, const int kind, PendingSegment *made) -> bool {
        const int W = kind == 2 ? 1 : wideW;
        const int U = kind == 2 ? afir_target::kSpecElementUnroll : kind == 1 ? 1 : shape.unroll;
        const bool slim = kind == 1;
        afir::RegionGeometry g;
        uint32_t rc = finish(afir::plan_fused_region(ra, W * U, block_dim, &g));
        if (rc != AFIR_HIP_OK) { failed = rc; return false; }
        if (g.empty) { skip = true; return false; }
        afir_target::SpecArgs sa;
        std::memset(&sa, 0, sizeof sa);
        for (int k = 0; k < 3; ++k) sa.size[k] = ra.size[k];
        sa.out = ra.out;
        sa.error_flag = ra.error_flag;
        sa.out_vec = ra.out_vec;
        afir_target::specExtentConstants(r->program, segment, res.shapes, sa.extent_const);
        sa.lanes_log2 = g.lanes_log2;
        sa.grid = (int)g.blocks;
        sa.column_blocks = (int)g.column_blocks;
        // vectors: every 128-bit access is aligned and rows are whole vectors; whole: no pass has a tail
        bool vectors, whole;
        int row_groups = 0;
        if (tile.tiled) {
          // one workgroup pass per tile of tile_p x tile_q
          const int64_t tq = (ra.size[last] + emit.tileQ - 1) / emit.tileQ;
          const int64_t tp = (ra.size[tile.dim] + emit.tileP - 1) / emit.tileP;
          int64_t tiles = tq * tp;
          for (int k = 0; k < last; ++k)
            if (k != tile.dim) tiles *= ra.size[k];
          int64_t blocks = tiles < (int64_t)afir::device_cus() * 256 ? tiles : (int64_t)afir::device_cus() * 256;
          if (block_dim) blocks = block_dim;
          sa.grid = (int)blocks;
          sa.column_blocks = 1;
          vectors = ra.out_vec != 0;
          whole = ra.size[last] % emit.tileQ == 0 && ra.size[tile.dim] % emit.tileP == 0;
        } else {
          // the aligned variant has no tail handling: whole groups, whole passes
          const int64_t groups = ra.size[last] / W;
          if (seg.reduce) {
            // lanes of a wavefront that share a row: enough for one pass over a short row, the wavefront otherwise
            const int64_t all_groups = (ra.size[last] + W - 1) / W;
            int ll = 0;
            while (ll < 6 && ((int64_t)U << ll) < all_groups) ++ll;
            sa.lanes_log2 = ll;
            if (!block_dim) {
              int64_t nrows = 1;
              for (int k = 0; k < last; ++k) nrows *= ra.size[k];
              const int64_t rows_per_block = (int64_t)4 * (64 >> ll);
              int64_t blocks = (nrows + rows_per_block - 1) / rows_per_block;
              if (blocks > (int64_t)afir::device_cus() * 16) blocks = (int64_t)afir::device_cus() * 16;
              sa.grid = (int)blocks;
            }
          }
          const int64_t per_pass = ((int64_t)1 << sa.lanes_log2) * U;
          vectors = ra.size[last] % W == 0 && (seg.reduce || ra.out_vec);
          if (!seg.reduce && !ra.out_vec) unaligned = true;
          whole = groups % per_pass == 0;
          // a row that fills a workgroup of 256 lanes with U groups each: a workgroup per row
          if (!slim && seg.reduce && groups == (int64_t)256 * U) row_groups = 1;
          // few rows of several such stretches: a workgroup per row as well, pass by pass
          int64_t nrows_all = 1;
          for (int k = 0; k < last; ++k) nrows_all *= ra.size[k];
          if (!slim && seg.reduce && groups >= (int64_t)512 * U && groups % ((int64_t)256 * U) == 0 &&
              nrows_all < (int64_t)afir::device_cus() * 16)
            row_groups = 2;
          // a handful of rows: the passes of a row are dealt out to about eight workgroups per CU in all
          const int64_t passes = groups / ((int64_t)256 * U);
          if (row_groups == 2 && nrows_all <= 64 && passes >= 8 && !block_dim) {
            int64_t per_row = (int64_t)afir::device_cus() * 8 / nrows_all;
            if (per_row > passes / 2) per_row = passes / 2;
            if (per_row >= 2 && per_row * nrows_all <= afir_target::kSpecPartials) {
              row_groups = 3;
              sa.column_blocks = (int)per_row;
            }
          }
        }
        for (int i = 0; i < ra.ninputs; ++i) {
          const afir::RegionInput &d = ra.in[i];
          afir_target::SpecInput &t = sa.in[i];
          t.base = d.base;
          t.index = d.index;
          for (int k = 0; k < 3; ++k) t.stride[k] = d.stride[k];
          t.offset = d.offset;
          t.gstride = d.gstride;
          t.gextent = d.gextent;
          t.vec = d.vec;
          t.gvec = d.gvec;
          if (tile.tiled && ((tile.inputs >> i) & 1u)) {
            // staged through LDS: 128-bit loads run along the tile dim
            const int64_t es = (int64_t)afir_region::elemTypeBytes(seg.inputs[i].type);
            bool tvec = aligned(d.base, d.offset * es);
            for (int k = 0; k < seg.rank; ++k)
              if (k != tile.dim && ra.size[k] > 1 && (d.stride[k] * es) % 16 != 0) tvec = false;
            t.vec = tvec ? 1 : 0;
            if (!tvec) vectors = false;
            continue;
          }
          // operands that are contiguous along the innermost dim are read with
          // 128-bit loads by the aligned variant
          if (d.stride[last] == 1 && d.gdim != last && (!d.vec || (d.gdim >= 0 && !d.gvec))) {
            vectors = false;
            unaligned = true;
          }
        }
        const int mode = kind == 2 ? afir_target::kSpecGeneral
                         : vectors && whole ? afir_target::kSpecAligned
                         : vectors && !tile.tiled ? afir_target::kSpecVector : afir_target::kSpecGeneral;
        if (kind == 2) row_groups = 0;
        if (row_groups == 3 && mode == afir_target::kSpecAligned) {
          int64_t nrows = 1;
          for (int k = 0; k < last; ++k) nrows *= ra.size[k];
          sa.grid = (int)(nrows * sa.column_blocks);
        } else if (row_groups && mode == afir_target::kSpecAligned) {
          // up to 16 workgroups per CU walk the rows (4 to 16 measured within 1 %, 2 slower)
          int64_t nrows = 1;
          for (int k = 0; k < last; ++k) nrows *= ra.size[k];
          int64_t blocks = nrows < (int64_t)afir::device_cus() * 16 ? nrows : (int64_t)afir::device_cus() * 16;
          if (block_dim) blocks = block_dim;
          sa.grid = (int)blocks;
          sa.column_blocks = 1;
        } else {
          if (row_groups == 3) sa.column_blocks = 1;
          row_groups = 0;
        }
        if (slim && (!g.idx32 || mode == afir_target::kSpecGeneral)) return false;
        *made = PendingSegment{segment, sa, g.idx32, mode, row_groups, slim, kind == 2};
        return true;
      };
      // The kernel that separates the chip's reads from its writes: every lane of the launch
      // resident at once (eight workgroups of 256 lanes per compute unit, eight 16-byte groups
      // per lane: 64 MiB of output per launch, up to two launches), for shapes of whole
      // workgroups whose accesses are all aligned.  Anything else: the kernels below.
      auto prepare_phased = [&]() -> bool {
        if (block_dim || tile.tiled || seg.reduce || !afir::phased_enabled()) return false;
        if (const char *env = std::getenv("AFIR_HIP_REGION_PHASED"))
          if (env[0] == '0') return false;
        {
          std::lock_guard<std::mutex> lock(compiled->mutex);
          if (compiled->phased.empty())
            for (size_t k = 0; k < r->program.segments.size(); ++k)
              compiled->phased.push_back(afir_target::specPhased(r->program, (int)k));
        }
        const afir_target::SpecPhased ph = compiled->phased[segment];
        if (!ph.eligible) return false;
        const int last = seg.rank - 1;
        const int W = 16 / ph.elemBytes, G = afir_target::kSpecPhasedGroups;
        const int64_t n = a.size[last];
        if (n <= 0 || n % W != 0 || !a.out_vec) return false;
        for (int i = 0; i < a.ninputs; ++i) {
          const afir::RegionInput &d = a.in[i];
          if (d.stride[last] == 0) continue;   // one value per row
          if (d.stride[last] != 1 || !d.vec || (d.gdim >= 0 && !d.gvec)) return false;
        }
        int64_t nrows = 1;
        for (int k = 0; k < last; ++k) nrows *= a.size[k];
        const int64_t gpr = n / W;   // groups per row
        int ll = 0;
        int64_t cblocks = 1, blocks = 0;
        if (gpr % G == 0 && gpr / G <= 256 && ((gpr / G) & (gpr / G - 1)) == 0) {
          while (((int64_t)1 << ll) < gpr / G) ++ll;
          const int64_t rows_per_block = 256 >> ll;
          if (nrows % rows_per_block != 0) return false;
          blocks = nrows / rows_per_block;
        } else if (gpr % (256 * G) == 0 && ph.vectors == 0) {
          ll = 8;
          cblocks = gpr / (256 * G);
          blocks = nrows * cblocks;
        } else {
          return false;
        }
        const int64_t lds = (int64_t)ph.vectors * n * ph.elemBytes;
        if (lds > 16 * 1024) return false;
        afir::RegionGeometry g;
        if (afir::plan_fused_region(a, W * 4, 0, &g).code != 0 || g.empty || !g.idx32) return false;
        const std::string name = afir_target::specPhasedKernelName(segment);
        if (resident_per_cu(name, (unsigned)lds) < 8) return false;
        const int64_t capacity = (int64_t)afir::device_cus() * 8;
        if (blocks < (int64_t)afir::device_cus() * 2 || blocks > afir::kPhaseMaxLaunches * capacity) return false;
        const int64_t launches = (blocks + capacity - 1) / capacity;
        const int64_t take = (blocks + launches - 1) / launches;
        for (int64_t b0 = 0; b0 < blocks; b0 += take) {
          const int64_t nb = blocks - b0 < take ? blocks - b0 : take;
          afir_target::SpecArgs sa;
          std::memset(&sa, 0, sizeof sa);
          for (int k = 0; k < 3; ++k) sa.size[k] = a.size[k];
          sa.out = a.out;
          sa.error_flag = a.error_flag;
          sa.out_vec = 1;
          afir_target::specExtentConstants(r->program, segment, res.shapes, sa.extent_const);
          sa.lanes_log2 = ll;
          sa.grid = (int)nb;
          sa.column_blocks = (int)cblocks;
          sa.first_block = (int)b0;
          for (int i = 0; i < a.ninputs; ++i) {
            const afir::RegionInput &d = a.in[i];
            afir_target::SpecInput &t = sa.in[i];
            t.base = d.base;
            t.index = d.index;
            for (int k = 0; k < 3; ++k) t.stride[k] = d.stride[k];
            t.offset = d.offset;
            t.gstride = d.gstride;
            t.gextent = d.gextent;
            t.vec = d.vec;
            t.gvec = d.gvec;
          }
          PendingSegment made{segment, sa, true, afir_target::kSpecAligned, 0, false, false};
          made.lds = (unsigned)lds;
          made.phased = true;
          made.phased_bytes = nb * 256 * G * 16 * ph.streamed;
          bool gathered = false;
          for (int i = 0; i < a.ninputs; ++i) gathered = gathered || a.in[i].gdim >= 0;
          made.phased_rate = region_hold_rate(gathered, ph.streamed);
          made.args.hold_ticks = afir::phase_hold_ticks(made.phased_bytes, region_hold_base_ns, made.phased_rate);
          pending.push_back(made);
        }
        return true;
      };
      if (prepare_phased()) continue;
      PendingSegment made;
      bool ok = false;
      // A single row whose length is no multiple of the vector width (a rank-1 tensor, mostly): the
      // whole vectors go to the aligned kernels and the last few elements to the element kernel, two
      // launches, instead of everything to the general kernel.
      const int64_t n_last = seg.size[seg.rank - 1];
      // (only where the row is long enough for the second launch to be worth its few microseconds)
      bool single_row = !tile.tiled && !seg.reduce && n_last >= (int64_t)1 << 18 && n_last % wideW != 0;
      for (int k = 0; k + 1 < seg.rank; ++k) single_row = single_row && seg.size[k] == 1;
      for (int i = 0; i < a.ninputs; ++i) single_row = single_row && a.in[i].gdim != seg.rank - 1;
      if (single_row) {
        afir::RegionArgs head = a, tail = a;
        const int64_t whole_part = n_last - n_last % wideW;
        head.size[seg.rank - 1] = whole_part;
        tail.size[seg.rank - 1] = n_last - whole_part;
        tail.out = static_cast<char *>(a.out) + whole_part * (int64_t)afir_region::elemTypeBytes(seg.outType);
        for (int i = 0; i < a.ninputs; ++i) tail.in[i].offset += a.in[i].stride[seg.rank - 1] * whole_part;
        PendingSegment first, second;
        bool ok1 = whole_part / wideW < (int64_t)8 * shape.unroll && shape.unroll > 1 && prepare(head, 1, &first);
        if (!ok1 && failed == AFIR_HIP_OK) ok1 = prepare(head, 0, &first);
        const bool ok2 = ok1 && failed == AFIR_HIP_OK && first.mode != afir_target::kSpecGeneral && prepare(tail, 2, &second);
        if (failed != AFIR_HIP_OK) return failed;
        if (ok1 && ok2) {
          pending.push_back(first);
          pending.push_back(second);
          continue;
        }
        skip = false;   // not this way: as one piece below
      }
      if (!tile.tiled && shape.unroll > 1 && row_groups_all < (int64_t)8 * shape.unroll) ok = prepare(a, 1, &made);
      if (!ok && !skip && failed == AFIR_HIP_OK) ok = prepare(a, 0, &made);
      // rows off 16-byte boundaries: element accesses either way, so let consecutive lanes take
      // consecutive elements
      if (ok && !tile.tiled && unaligned && made.mode == afir_target::kSpecGeneral && !made.slim) ok = prepare(a, 2, &made);
      if (failed != AFIR_HIP_OK) return failed;
      // a gather along the innermost dim from contiguous, aligned source rows that fit the LDS: a
      // workgroup per row stages the source row and gathers from there
      if (ok && !made.slim && !made.elem && made.mode != afir_target::kSpecGeneral) {
        const afir_target::SpecStage stage = afir_target::specStage(r->program, segment);
        if (stage.input >= 0) {
          const afir::RegionInput &d = a.in[stage.input];
          const int64_t bytes = d.gextent * stage.elemBytes;
          const int64_t n_out = seg.size[seg.rank - 1];
          const int64_t wave_pass = (int64_t)64 * shape.unroll * wideW;     // elements a wavefront covers per pass
          // Output rows of half a pass to eight passes of a wavefront, a thousand rows or more, source
          // rows of at most 8 KiB: a wavefront per row, four rows per workgroup, each with its own part
          // of the LDS and no barriers (measured against a workgroup per row, f16, TB/s written:
          // [32768, 4096] from 1024 columns 1.15 -> 3.16, [16384, 2048] 1.56 -> 2.43, [2048, 16384]
          // 2.22 -> 2.82, [16384, 8192] from 4096 columns equal; slower with 16 KiB source rows, which
          // leave two workgroups per CU, and with fewer rows than the chip has wavefront slots)
          if (d.gstride == 1 && d.vec && bytes > 0 && bytes % 16 == 0 && bytes * 4 <= afir_target::kSpecStageBytes / 2 &&
              n_out * 2 >= wave_pass && n_out <= 8 * wave_pass && seg.size[0] >= 1024) {
            int64_t blocks = (seg.size[0] + 3) / 4;
            if (blocks > (int64_t)afir::device_cus() * 16) blocks = (int64_t)afir::device_cus() * 16;
            if (block_dim) blocks = block_dim;
            made.args.grid = (int)blocks;
            made.args.column_blocks = 1;
            made.lds = (unsigned)(bytes * 4);
            made.stage_wave = true;
            if (made.mode == afir_target::kSpecAligned && (n_out / wideW) % ((int64_t)64 * shape.unroll) != 0)
              made.mode = afir_target::kSpecVector;
          } else
          if (d.gstride == 1 && d.vec && bytes > 0 && bytes % 16 == 0 && bytes <= afir_target::kSpecStageBytes &&
              seg.size[seg.rank - 1] >= (int64_t)128 * shape.unroll * wideW) {   // at least half a pass of the workgroup
            int64_t blocks = seg.size[0] < (int64_t)afir::device_cus() * 16 ? seg.size[0] : (int64_t)afir::device_cus() * 16;
            if (block_dim) blocks = block_dim;
            made.args.grid = (int)blocks;
            made.args.column_blocks = 1;
            made.lds = (unsigned)bytes;
            const int64_t per_pass = (int64_t)256 * shape.unroll;     // the whole workgroup on a row
            if (made.mode == afir_target::kSpecAligned && (seg.size[seg.rank - 1] / wideW) % per_pass != 0)
              made.mode = afir_target::kSpecVector;
          }
        }
      }
      if (ok) pending.push_back(made);
      continue;
    }
    uint32_t rc = finish(afir::launch_fused_region(a, block_dim, static_cast<hipStream_t>(stream)));
    if (rc != AFIR_HIP_OK) return rc;
  }
  if (!pending.empty()) {
    auto launch = [&](const std::string &name, void *args, size_t bytes, unsigned blocks, unsigned lds = 0) -> uint32_t {
      hipFunction_t fn = nullptr;
      const std::string no = compiled_function(compiled.get(), r->program, name, &fn);
      if (!no.empty()) return fail(AFIR_HIP_E_LAUNCH, no);
      void *config[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, args, HIP_LAUNCH_PARAM_BUFFER_SIZE, &bytes, HIP_LAUNCH_PARAM_END};
      thread_local std::string launched;   // the note keeps a pointer to the name
      launched = name;
      afir::last_launch_note() = afir::LaunchNote{launched.c_str(), blocks, 256u};
      const hipError_t e = hipModuleLaunchKernel(fn, blocks, 1, 1, 256, 1, 1, lds, static_cast<hipStream_t>(stream),
                                                 nullptr, config);
      if (e != hipSuccess) return fail(AFIR_HIP_E_LAUNCH, std::string("compiled region kernel: ") + hipGetErrorString(e));
      return AFIR_HIP_OK;
    };
    // segments that agree on the kernel variant go out as one launch
    const int nseg = (int)res.segments.size();
    bool together = pending.size() > 1 && nseg <= afir_target::kSpecMaxSegments;
    // ... also those that separate reads from writes, when one launch of all of them is still
    // resident at once: the hold is then that of everything the launch reads
    bool together_phased = together;
    int64_t total = 0, phased_bytes = 0;
    double phased_ns = 0;   // the segments' reads one after the other, each at its rate
    unsigned phased_lds = 0;
    for (const PendingSegment &p : pending) {
      together = together && p.idx32 == pending[0].idx32 && p.mode == pending[0].mode && !p.rows && !p.slim && !p.elem &&
                 !p.lds && !p.phased;
      together_phased = together_phased && p.phased && p.args.first_block == 0 &&
                        (&p == &pending[0] || p.segment != (&p)[-1].segment);
      total += p.args.grid;
      phased_bytes += p.phased_bytes;
      if (p.phased_rate) phased_ns += (double)p.phased_bytes / p.phased_rate;
      phased_lds = p.lds > phased_lds ? p.lds : phased_lds;
    }
    together_phased = together_phased && total <= (int64_t)afir::device_cus() * 8 &&
                      resident_per_cu(afir_target::specAllPhasedKernelName(), phased_lds) >= 8;
    if (together_phased) {
      afir_target::SpecAll all;
      std::memset(&all, 0, sizeof all);
      int next = 0;
      size_t at = 0;
      for (int k = 0; k < nseg; ++k) {
        all.first[k] = next;
        if (at < pending.size() && pending[at].segment == k) {
          all.seg[k] = pending[at].args;
          all.seg[k].hold_ticks = afir::phase_hold_ticks(
              phased_bytes, region_hold_base_ns, phased_ns > 0 ? (int)((double)phased_bytes / phased_ns) : 6900);
          next += pending[at].args.grid;
          ++at;
        }
      }
      for (int k = nseg; k <= afir_target::kSpecMaxSegments; ++k) all.first[k] = next;
      const uint32_t rc = launch(afir_target::specAllPhasedKernelName(), &all,
                                 offsetof(afir_target::SpecAll, seg) + (size_t)nseg * sizeof(afir_target::SpecArgs),
                                 (unsigned)next, phased_lds);
      if (rc != AFIR_HIP_OK) return rc;
    } else if (together && total <= 0x7fffffff) {
      afir_target::SpecAll all;
      std::memset(&all, 0, sizeof all);
      int next = 0;
      size_t at = 0;
      for (int k = 0; k < nseg; ++k) {
        all.first[k] = next;
        if (at < pending.size() && pending[at].segment == k) {
          all.seg[k] = pending[at].args;
          next += pending[at].args.grid;
          ++at;
        }
      }
      for (int k = nseg; k <= afir_target::kSpecMaxSegments; ++k) all.first[k] = next;
      const uint32_t rc = launch(afir_target::specAllKernelName(pending[0].idx32, pending[0].mode), &all,
                                 offsetof(afir_target::SpecAll, seg) + (size_t)nseg * sizeof(afir_target::SpecArgs),
                                 (unsigned)next);
      if (rc != AFIR_HIP_OK) return rc;
    } else {
      for (PendingSegment &p : pending) {
        if (p.rows == 3) {
          // split and join share the code object's partial sums with every other launch of this
          // form: order them (a launch on another stream waits for the previous join)
          CompiledRegion *c = compiled.get();
          std::lock_guard<std::mutex> chain(c->split_mutex);
          hipStream_t st = static_cast<hipStream_t>(stream);
          if (!c->split_done && hipEventCreateWithFlags(&c->split_done, hipEventDisableTiming) != hipSuccess) {
            (void)hipGetLastError();
            return fail(AFIR_HIP_E_LAUNCH, "compiled region kernel: cannot create the event that orders split row sums");
          }
          if (c->split_recorded && c->split_stream != st && hipStreamWaitEvent(st, c->split_done, 0) != hipSuccess) {
            (void)hipGetLastError();
            return fail(AFIR_HIP_E_LAUNCH, "compiled region kernel: cannot order split row sums across streams");
          }
          uint32_t rc = launch(afir_target::specSplitRowsKernelName(p.segment, p.idx32, false), &p.args, sizeof p.args,
                               (unsigned)p.args.grid);
          if (rc != AFIR_HIP_OK) return rc;
          const int64_t nrows = p.args.grid / p.args.column_blocks;
          rc = launch(afir_target::specSplitRowsKernelName(p.segment, p.idx32, true), &p.args, sizeof p.args,
                      (unsigned)((nrows + 3) / 4));
          if (rc != AFIR_HIP_OK) return rc;
          if (hipEventRecord(c->split_done, st) != hipSuccess) {
            (void)hipGetLastError();
            return fail(AFIR_HIP_E_LAUNCH, "compiled region kernel: cannot record the event that orders split row sums");
          }
          c->split_recorded = true;
          c->split_stream = st;
          continue;
        }
        if (p.phased) {
          const uint32_t rc = launch(afir_target::specPhasedKernelName(p.segment), &p.args, sizeof p.args,
                                     (unsigned)p.args.grid, p.lds);
          if (rc != AFIR_HIP_OK) return rc;
          continue;
        }
        if (p.lds) {
          const uint32_t rc = launch(afir_target::specStagedKernelName(p.segment, p.idx32, p.mode, p.stage_wave), &p.args, sizeof p.args,
                                     (unsigned)p.args.grid, p.lds);
          if (rc != AFIR_HIP_OK) return rc;
          continue;
        }
        const uint32_t rc = launch(p.rows == 2 ? afir_target::specLongRowsKernelName(p.segment, p.idx32)
                                   : p.rows ? afir_target::specRowsKernelName(p.segment, p.idx32)
                                   : p.elem ? afir_target::specElementKernelName(p.segment, p.idx32)
                                   : p.slim ? afir_target::specSlimKernelName(p.segment, p.mode)
                                            : afir_target::specKernelName(p.segment, p.idx32, p.mode),
                                   &p.args, sizeof p.args, (unsigned)p.args.grid);
        if (rc != AFIR_HIP_OK) return rc;
      }
    }
  }
  g_last_error.clear();
  return AFIR_HIP_OK;
}

int afir_hip_kernel_count(void) { return kNumKernels; }

const char *afir_hip_family_program(const char *family) {
  if (!family) return nullptr;
  for (const FamilyRegion &f : g_families)
    if (std::strcmp(f.name, family) == 0) return f.program;
  return nullptr;
}

const AfirHipKernelInfo *afir_hip_kernel_info(int index) {
  if (index < 0 || index >= kNumKernels) return nullptr;
  return &kKernels[index];
}

const AfirHipKernelInfo *afir_hip_find_kernel(const char *name) {
  if (!name) return nullptr;
  for (int i = 0; i < kNumKernels; ++i)
    if (std::strcmp(kKernels[i].name, name) == 0) return &kKernels[i];
  return nullptr;
}

uint32_t afir_hip_argument_bytes(const char *kernel_name, const void *tiling, size_t tiling_len,
                                 size_t *bytes, int max_args) {
  const AfirHipKernelInfo *info = afir_hip_find_kernel(kernel_name);
  if (!info)
    return fail(AFIR_HIP_E_UNKNOWN,
                std::string("no fused kernel named '") + (kernel_name ? kernel_name : "") + "'");
  const int nargs = info->num_inputs + info->num_outputs;
  if (!bytes || max_args < nargs) return fail(AFIR_HIP_E_INVALID, "argument_bytes: output array too small");
  const size_t want_len = sizeof(int64_t) * (size_t)info->num_tiling_fields;
  if (!tiling || tiling_len != want_len) {
    char buf[160];
    std::snprintf(buf, sizeof buf, "%s: tiling data must be %zu bytes (%d int64 fields), got %zu",
                  info->name, want_len, info->num_tiling_fields, tiling_len);
    return fail(AFIR_HIP_E_INVALID, buf);
  }
  int64_t f[4] = {0, 0, 0, 0};
  std::memcpy(f, tiling, want_len);
  const int dims = info->num_tiling_fields - ((info - kKernels) == 4 ? 1 : 0);
  for (int i = 0; i < dims; ++i)
    if (f[i] < 0 || f[i] > (int64_t)1 << 40)
      return fail(AFIR_HIP_E_INVALID, std::string(info->name) + ": extent out of range in tiling data");
  auto sz = [](int64_t a, int64_t b, int64_t c, int64_t elem) {
    return (size_t)((unsigned __int128)a * (unsigned __int128)b * (unsigned __int128)c * (unsigned __int128)elem);
  };
  switch ((int)(info - kKernels)) {
    case 0: bytes[0] = bytes[1] = bytes[2] = sz(f[0], f[1], 1, 4); break;
    case 1: bytes[0] = sz(f[0], f[1], 1, 4); bytes[1] = sz(f[1], 1, 1, 4); bytes[2] = sz(f[0], 1, 1, 4); break;
    case 2: bytes[0] = bytes[2] = sz(f[0], f[1], f[2], 2); bytes[1] = sz(f[2], 1, 1, 2); break;
    case 3:
      bytes[0] = sz(f[0], f[1], 1, 2); bytes[1] = sz(f[2], 1, 1, 4);
      bytes[2] = bytes[3] = sz(f[1], 1, 1, 2); bytes[4] = sz(f[2], f[1], 1, 2);
      break;
    case 4:
      bytes[0] = sz(f[0], f[1], 1, 2); bytes[1] = sz(f[1], f[2], 1, 2);
      bytes[2] = sz(f[2], 1, 1, 2); bytes[3] = sz(f[0], f[2], 1, 2);
      break;
  }
  g_last_error.clear();
  return AFIR_HIP_OK;
}

uint32_t afir_hip_launch(const char *kernel_name, uint32_t block_dim, void *stream, int num_args,
                         void *const *args, void *workspace, const void *tiling,
                         size_t tiling_len) {
  const AfirHipKernelInfo *info = afir_hip_find_kernel(kernel_name);
  if (!info)
    return fail(AFIR_HIP_E_UNKNOWN,
                std::string("no fused kernel named '") + (kernel_name ? kernel_name : "") + "'");
  const int want = info->num_inputs + info->num_outputs;
  if (num_args != want || (want > 0 && !args)) {
    char buf[160];
    std::snprintf(buf, sizeof buf, "%s: expected %d tensor arguments (%d inputs, %d outputs), got %d",
                  info->name, want, info->num_inputs, info->num_outputs, num_args);
    return fail(AFIR_HIP_E_INVALID, buf);
  }
  const size_t want_len = sizeof(int64_t) * (size_t)info->num_tiling_fields;
  if (!tiling || tiling_len != want_len) {
    char buf[160];
    std::snprintf(buf, sizeof buf, "%s: tiling data must be %zu bytes (%d int64 fields), got %zu",
                  info->name, want_len, info->num_tiling_fields, tiling_len);
    return fail(AFIR_HIP_E_INVALID, buf);
  }
  void *tl = const_cast<void *>(tiling);
  const int idx = (int)(info - kKernels);
  switch (idx) {
    case 0:
      return afir_hip_launch_fused_add_mul(block_dim, stream, args[0], args[1], args[2], workspace, tl);
    case 1:
      return afir_hip_launch_broadcast_add_reducesum(block_dim, stream, args[0], args[1], args[2],
                                                     workspace, tl);
    case 2:
      return afir_hip_launch_relu_broadcast_add_transpose(block_dim, stream, args[0], args[1],
                                                          args[2], workspace, tl);
    case 3:
      return afir_hip_launch_gather_scale_shift(block_dim, stream, args[0], args[1], args[2],
                                                args[3], args[4], workspace, tl);
    case 4:
      return afir_hip_launch_matmul_add_leakyrelu(block_dim, stream, args[0], args[1], args[2],
                                                  args[3], workspace, tl);
  }
  return fail(AFIR_HIP_E_UNKNOWN, "unreachable");
}

}  // extern "C"
