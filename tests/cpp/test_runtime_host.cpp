// Host-only checks of the runtime's on-disk formats and comparator against the
// known answers the reference's own tests hold:
//   npy        test/tools/runtime/test_runtime.cpp:169-323
//   tiling     test/tools/runtime/test_tiling_schema.cpp:80-117,176-199
//   comparator test/tools/runtime/test_taskgraph_runtime.cpp:1773-1863
// Built and run by tests/test_runtime_host.py (no GPU needed).
#include <cmath>
#include <cstdio>
#include <cstring>
#include <fstream>
#include <string>
#include <vector>

#include "runtime.h"

using namespace afirt;

// The GPU runner is not linked into this host-only binary; nothing here runs a kernel.
std::unique_ptr<ExecutionRunner> afirt::createHipExecutionRunner() { return nullptr; }

static int g_pass = 0, g_fail = 0;
#define EXPECT(cond, msg)                                   \
  do {                                                      \
    if (cond) { ++g_pass; }                                 \
    else { ++g_fail; std::printf("FAIL: %s (%s:%d)\n", msg, __FILE__, __LINE__); } \
  } while (0)

static std::string g_tmp;

static void writeNpy(const std::string &path, const char *descr, const std::vector<int64_t> &shape,
                     const void *data, size_t bytes) {
  std::string sh = "(";
  for (size_t i = 0; i < shape.size(); ++i) {
    sh += std::to_string(shape[i]);
    if (shape.size() == 1 || i + 1 < shape.size()) sh += ",";
  }
  sh += ")";
  std::string dict = std::string("{'descr': '") + descr + "', 'fortran_order': False, 'shape': " + sh + ", }";
  size_t total = 10 + dict.size() + 1;
  dict.append((64 - total % 64) % 64, ' ');
  dict += '\n';
  uint16_t hlen = (uint16_t)dict.size();
  std::ofstream f(path, std::ios::binary);
  f.write("\x93NUMPY", 6);
  f.put(1);
  f.put(0);
  f.write(reinterpret_cast<char *>(&hlen), 2);
  f.write(dict.data(), (std::streamsize)dict.size());
  f.write(static_cast<const char *>(data), (std::streamsize)bytes);
}

static void testNpy() {
  {  // f16 1.0 = 0x3C00
    std::vector<uint16_t> v = {0x3C00, 0x4000, 0x0000};
    writeNpy(g_tmp + "/f16.npy", "<f2", {3}, v.data(), 6);
    auto r = LoadNpy(g_tmp + "/f16.npy");
    EXPECT((bool)r, "f16 loads");
    if (r) {
      EXPECT(r->dtype == DType::F16, "f16 dtype");
      EXPECT(r->shape == std::vector<int64_t>{3}, "f16 shape");
      uint16_t x;
      std::memcpy(&x, r->data, 2);
      EXPECT(x == 0x3C00, "f16 data[0]");
      EXPECT(SaveNpy(g_tmp + "/f16_out.npy", *r).ok(), "f16 saves");
    }
  }
  {  // bf16 1.0 = 0x3F80, stored as <V2
    std::vector<uint16_t> v = {0x3F80, 0x4000, 0x0000};
    writeNpy(g_tmp + "/bf16.npy", "<V2", {3}, v.data(), 6);
    auto r = LoadNpy(g_tmp + "/bf16.npy");
    EXPECT((bool)r, "bf16 loads");
    if (r) {
      EXPECT(r->dtype == DType::BF16, "bf16 dtype");
      EXPECT(SaveNpy(g_tmp + "/bf16_out.npy", *r).ok(), "bf16 saves");
      auto r2 = LoadNpy(g_tmp + "/bf16_out.npy");
      EXPECT((bool)r2 && r2->dtype == DType::BF16, "bf16 round trip dtype");
      if (r2) {
        uint16_t x;
        std::memcpy(&x, r2->data, 2);
        EXPECT(x == 0x3F80, "bf16 round trip data[0]");
      }
    }
  }
  {
    std::vector<float> v = {1.f, 2.f, 3.f, 4.f};
    writeNpy(g_tmp + "/f32.npy", "<f4", {4}, v.data(), 16);
    auto r = LoadNpy(g_tmp + "/f32.npy");
    EXPECT((bool)r && r->dtype == DType::F32, "f32 loads");
    if (r) {
      float x;
      std::memcpy(&x, r->data, 4);
      EXPECT(x == 1.0f, "f32 data[0]");
    }
  }
  {
    std::vector<int8_t> v = {1, -2, 127, -128};
    writeNpy(g_tmp + "/i8.npy", "|i1", {4}, v.data(), 4);
    auto r = LoadNpy(g_tmp + "/i8.npy");
    EXPECT((bool)r && r->dtype == DType::INT8 && r->nbytes() == 4, "i8 loads");
    if (r) EXPECT(SaveNpy(g_tmp + "/i8_out.npy", *r).ok(), "i8 saves");
  }
  {
    std::vector<int32_t> v = {100, -200, 0, 2147483647};
    writeNpy(g_tmp + "/i32.npy", "<i4", {4}, v.data(), 16);
    auto r = LoadNpy(g_tmp + "/i32.npy");
    EXPECT((bool)r && r->dtype == DType::INT32, "i32 loads");
  }
  {
    std::vector<int64_t> v = {1000000LL, -2000000LL, 0};
    writeNpy(g_tmp + "/i64.npy", "<i8", {3}, v.data(), 24);
    auto r = LoadNpy(g_tmp + "/i64.npy");
    EXPECT((bool)r && r->dtype == DType::INT64 && r->nbytes() == 24, "i64 loads");
    if (r) {
      int64_t x;
      std::memcpy(&x, r->data, 8);
      EXPECT(x == 1000000LL, "i64 data[0]");
    }
  }
  {  // 2-D and header padding rule
    std::vector<float> v(6, 1.5f);
    NDArray a;
    a.dtype = DType::F32;
    a.shape = {2, 3};
    a.setExternal(v.data());
    EXPECT(SaveNpy(g_tmp + "/m.npy", a).ok(), "2-D saves");
    std::ifstream f(g_tmp + "/m.npy", std::ios::binary);
    std::string raw((std::istreambuf_iterator<char>(f)), std::istreambuf_iterator<char>());
    uint16_t hlen;
    std::memcpy(&hlen, raw.data() + 8, 2);
    EXPECT((10 + hlen) % 64 == 0, "header padded to 64");
    EXPECT(raw[10 + hlen - 1] == '\n', "header newline terminated");
    EXPECT(raw.find("'shape': (2,3), }") != std::string::npos, "2-D shape text");
    auto r = LoadNpy(g_tmp + "/m.npy");
    EXPECT((bool)r && r->shape == (std::vector<int64_t>{2, 3}), "2-D shape round trip");
  }
  // errors
  {
    std::vector<double> v = {1.0, 2.0};
    writeNpy(g_tmp + "/f64.npy", "<f8", {2}, v.data(), 16);
    auto r = LoadNpy(g_tmp + "/f64.npy");
    EXPECT(!r && r.error().find("Unsupported dtype") != std::string::npos, "<f8 rejected");
    EXPECT(!LoadNpy(g_tmp + "/missing.npy"), "missing file rejected");
    std::vector<float> one = {1.f};
    writeNpy(g_tmp + "/trunc.npy", "<f4", {3}, one.data(), 4);
    auto t = LoadNpy(g_tmp + "/trunc.npy");
    EXPECT(!t && t.error().find("Truncated") != std::string::npos, "truncated payload rejected");
    std::ofstream(g_tmp + "/junk.npy") << "not numpy at all";
    EXPECT(!LoadNpy(g_tmp + "/junk.npy"), "junk rejected");
  }
  {  // scalar: empty shape = one element
    NDArray a;
    a.dtype = DType::F32;
    EXPECT(a.numElements() == 1 && a.nbytes() == 4, "empty shape is a scalar");
  }
}

static void testTiling() {
  const std::string six = g_tmp + "/six.json";
  std::ofstream(six) << R"({"kernel":"k","tiling_params":[
    {"name":"TB_M","type":"int64","min":16,"max":16,"step":16},
    {"name":"TB_N","type":"int64","values":[16]},
    {"name":"dim_arg0_0","type":"int64","fixed":true},
    {"name":"dim_arg1_1","type":"int64","fixed":true},
    {"name":"dim_arg0_1","type":"int64","fixed":true},
    {"name":"dim_arg1_0","type":"int64","fixed":true}]})";
  auto s = TilingSchema::fromJson(six);
  EXPECT((bool)s, "fromJson succeeds");
  if (!s) return;
  EXPECT(s->size() == 6, "6 fields");
  EXPECT(s->fields()[0].name == "TB_M" && s->fields()[0].type == "int64", "field 0");
  EXPECT(s->fields()[5].name == "dim_arg1_0", "field 5");
  using P = std::pair<std::string, int64_t>;
  auto bytes = s->pack({P{"TB_M", 16}, P{"TB_N", 16}, P{"dim_arg0_0", 64}, P{"dim_arg1_1", 64},
                        P{"dim_arg0_1", 64}, P{"dim_arg1_0", 64}});
  EXPECT((bool)bytes && bytes->size() == 48, "6 x int64 = 48 bytes");
  if (bytes) {
    int64_t first, last;
    std::memcpy(&first, bytes->data(), 8);
    std::memcpy(&last, bytes->data() + 40, 8);
    EXPECT(first == 16 && last == 64, "first 16, last 64");
  }
  auto wrongCount = s->pack({P{"TB_M", 16}, P{"TB_N", 16}});
  EXPECT(!wrongCount && wrongCount.error().find("count mismatch") != std::string::npos, "count mismatch");
  auto wrongName = s->pack({P{"WRONG", 16}, P{"TB_N", 16}, P{"dim_arg0_0", 64}, P{"dim_arg1_1", 64},
                            P{"dim_arg0_1", 64}, P{"dim_arg1_0", 64}});
  EXPECT(!wrongName && wrongName.error().find("name mismatch") != std::string::npos &&
             wrongName.error().find("WRONG") != std::string::npos &&
             wrongName.error().find("TB_M") != std::string::npos,
         "name mismatch names both");
  EXPECT(!TilingSchema::fromJson("/nonexistent/schema.json"), "missing schema file");
  std::ofstream(g_tmp + "/bad.json") << "{ not valid json";
  EXPECT(!TilingSchema::fromJson(g_tmp + "/bad.json"), "malformed schema");
  std::ofstream(g_tmp + "/mixed.json") << R"({"tiling_params":[{"name":"A","type":"int64"},{"name":"B","type":"int32"},{"name":"C"}]})";
  auto m = TilingSchema::fromJson(g_tmp + "/mixed.json");
  EXPECT((bool)m && m->size() == 3 && m->fields()[2].type == "int64", "mixed schema, default type");
  if (m) {
    auto b = m->pack({P{"A", 1}, P{"B", 2}, P{"C", 3}});
    EXPECT((bool)b && b->size() == 20, "int64+int32+int64 = 20 bytes");
    if (b) {
      int64_t a, c;
      int32_t bb;
      std::memcpy(&a, b->data(), 8);
      std::memcpy(&bb, b->data() + 8, 4);
      std::memcpy(&c, b->data() + 12, 8);
      EXPECT(a == 1 && bb == 2 && c == 3, "1,2,3");
    }
  }
  // run-manifest form: named params in any order, schema order in the bytes
  TilingBinding tb;
  tb.schemaPath = six;
  tb.params = "dim_arg1_0=640,TB_M=16,TB_N=16,dim_arg0_0=640,dim_arg1_1=512,dim_arg0_1=1";
  auto packed = packTilingBytes(tb);
  EXPECT((bool)packed && packed->size() == 48, "named params pack");
  if (packed) {
    int64_t v[6];
    std::memcpy(v, packed->data(), 48);
    EXPECT(v[0] == 16 && v[2] == 640 && v[3] == 512 && v[4] == 1 && v[5] == 640, "schema order");
  }
  tb.params = "TB_M=16";
  auto missing = packTilingBytes(tb);
  EXPECT(!missing && missing.error().find("missing field") != std::string::npos, "missing field");
  tb.params = "TB_M";
  EXPECT(!packTilingBytes(tb), "token without '='");
  TilingBinding only;
  only.params = "A=1";
  EXPECT(!packTilingBytes(only), "params without schema or binary");
  EXPECT(packTilingBytes(std::nullopt)->empty(), "no tiling = empty bytes");
  TilingBinding bin;
  bin.binaryPath = g_tmp + "/t.bin";
  std::ofstream(bin.binaryPath, std::ios::binary) << std::string("\x01\x02\x03", 3);
  auto raw = packTilingBytes(bin);
  EXPECT((bool)raw && raw->size() == 3 && (*raw)[2] == 3, "binary tiling passes through");
}

static NDArray f32Array(std::vector<int64_t> shape, std::vector<float> v) {
  NDArray a;
  a.dtype = DType::F32;
  a.shape = std::move(shape);
  a.allocate();
  std::memcpy(a.data, v.data(), v.size() * 4);
  return a;
}

static void testComparator() {
  {
    std::vector<NDArray> a, e;
    a.push_back(f32Array({2}, {1.f, 2.f}));
    e.push_back(f32Array({2}, {1.f, 2.f}));
    auto r = compareRuntimeOutputs(a, e, 0.0, 0.0);
    EXPECT((bool)r && r->passed && r->maxAbsDiff == 0.0 && r->meanAbsDiff == 0.0 && r->errorMessage.empty(),
           "exact match passes at atol=rtol=0");
  }
  {
    std::vector<NDArray> a, e;
    a.push_back(f32Array({2}, {1.f, 2.25f}));
    e.push_back(f32Array({2}, {1.f, 2.f}));
    auto r = compareRuntimeOutputs(a, e, 1e-4, 1e-4);
    EXPECT((bool)r && !r->passed && r->maxAbsDiff > 0 && r->meanAbsDiff > 0 && !r->errorMessage.empty() &&
               r->mismatches == 1,
           "2.25 vs 2.0 fails at 1e-4");
    auto loose = compareRuntimeOutputs(a, e, 0.0, 0.2);
    EXPECT((bool)loose && loose->passed, "passes within rtol*|expected|");
  }
  {
    std::vector<NDArray> a, none;
    a.push_back(f32Array({2}, {1.f, 2.f}));
    auto r = compareRuntimeOutputs(a, none, 0, 0);
    EXPECT(!r && !r.error().empty(), "count mismatch is an error");
    std::vector<NDArray> e;
    e.push_back(f32Array({1, 2}, {1.f, 2.f}));
    EXPECT(!compareRuntimeOutputs(a, e, 0, 0), "shape mismatch is an error");
    std::vector<NDArray> ei;
    NDArray i32;
    i32.dtype = DType::INT32;
    i32.shape = {2};
    i32.allocate();
    ei.push_back(std::move(i32));
    EXPECT(!compareRuntimeOutputs(a, ei, 0, 0), "dtype mismatch is an error");
  }
  {  // half decodes: 0x3C00 and 0x3F80 are 1.0
    NDArray h, b, one;
    h.dtype = DType::F16; h.shape = {1}; h.allocate();
    uint16_t hv = 0x3C00; std::memcpy(h.data, &hv, 2);
    NDArray h2; h2.dtype = DType::F16; h2.shape = {1}; h2.allocate();
    uint16_t hv2 = 0x4000; std::memcpy(h2.data, &hv2, 2);
    std::vector<NDArray> a, e;
    a.push_back(std::move(h)); e.push_back(std::move(h2));
    auto r = compareRuntimeOutputs(a, e, 0, 0);
    EXPECT((bool)r && std::fabs(r->maxAbsDiff - 1.0) < 1e-12, "f16 1.0 vs 2.0 differ by 1");
    b.dtype = DType::BF16; b.shape = {1}; b.allocate();
    uint16_t bv = 0x3F80; std::memcpy(b.data, &bv, 2);
    one.dtype = DType::BF16; one.shape = {1}; one.allocate();
    uint16_t ov = 0x4000; std::memcpy(one.data, &ov, 2);
    std::vector<NDArray> a2, e2;
    a2.push_back(std::move(b)); e2.push_back(std::move(one));
    auto r2 = compareRuntimeOutputs(a2, e2, 0, 0);
    EXPECT((bool)r2 && std::fabs(r2->maxAbsDiff - 1.0) < 1e-12, "bf16 1.0 vs 2.0 differ by 1");
  }
}

static void testArtifactsAndManifests() {
  const std::string src = g_tmp + "/example.mlir";
  std::ofstream(src) << "func.func @example(%arg0: tensor<4x4xf32>, %arg1: tensor<4x4xf32>) -> tensor<4x4xf32> {\n"
                        "  %0 = afir.add %arg0, %arg1 : (tensor<4x4xf32>, tensor<4x4xf32>) -> tensor<4x4xf32>\n"
                        "  %1 = afir.mul %0, %arg1 : (tensor<4x4xf32>, tensor<4x4xf32>) -> tensor<4x4xf32>\n"
                        "  return %1 : tensor<4x4xf32>\n}\n";
  CompileRequest req;
  req.kernelSource = src;
  req.outputDir = g_tmp + "/art";
  auto a = compileArtifact(req);
  EXPECT((bool)a, "afir add->mul chain compiles");
  if (a) {
    EXPECT(a->kernelName == "example" && a->sharedLibrarySymbol == "afir_hip_launch_region" &&
               a->regionProgram.find("push arg1 d0 d1\nmul\n") != std::string::npos, "artifact fields");
    auto text = readTextFile(a->manifestPath);
    EXPECT((bool)text && text->find("kernel_name=example\n") != std::string::npos &&
               text->find("kernel_kind=vec\n") != std::string::npos &&
               text->find("device_binary_path=example.hipk\n") != std::string::npos &&
               text->find("manifest_path=out/manifest.txt\n") != std::string::npos,
           "manifest keys");
    auto back = loadArtifactFromRoot(g_tmp + "/art");
    EXPECT((bool)back && back->kernelName == "example" && back->sharedLibrarySymbol == a->sharedLibrarySymbol &&
               back->regionProgram == a->regionProgram,
           "artifact reloads");
  }
  // any AFIR chain lowers to a program; (a + b) * a keeps its own operand order
  auto other = compileSourceText("func.func @f(%a: tensor<4xf32>, %b: tensor<4xf32>) -> tensor<4xf32> {\n"
                                 "%0 = afir.add %a, %b : (tensor<4xf32>, tensor<4xf32>) -> tensor<4xf32>\n"
                                 "%1 = afir.mul %0, %a : (tensor<4xf32>, tensor<4xf32>) -> tensor<4xf32>\n"
                                 "return %1 : tensor<4xf32>\n}", "");
  EXPECT((bool)other && other->hipKernel == "fused_region" &&
             other->program.find("push arg0 d0\npush arg1 d0\nadd\npush arg0 d0\nmul\n") != std::string::npos,
         "(a+b)*a lowers as written");
  auto explicitFamily = compileSourceText("hip_kernel=gather_scale_shift\n", "");
  EXPECT((bool)explicitFamily && explicitFamily->hipKernel == "gather_scale_shift" &&
             explicitFamily->symbol == "afir_hip_launch_gather_scale_shift" && explicitFamily->program.empty(),
         "explicit family");
  EXPECT(!compileSourceText("hip_kernel=nope\n", ""), "unknown family rejected");
  EXPECT(!compileSourceText("hip_kernel=fused_region\n", ""), "a region needs a program, not a name");
  EXPECT(!compileSourceText("func.func @mystery() { return }", ""), "function without a tensor result rejected");
  auto unsupported = compileSourceText("func.func @f(%a: tensor<4xf32>) -> tensor<4xf32> {\n"
                                       "%0 = afir.exp %a : tensor<4xf32> -> tensor<4xf32>\nreturn %0 : tensor<4xf32>\n}", "");
  EXPECT(!unsupported && unsupported.error().find("line 2") != std::string::npos &&
             unsupported.error().find("afir.exp has no HIP lowering") != std::string::npos,
         "unsupported op is named with its line");
  {  // descriptor round trip with a program
    HipKernelDescriptor d = *other;
    d.kernelName = "k";
    auto back = parseDescriptor(serializeDescriptor(d));
    EXPECT((bool)back && back->program == d.program && back->hipKernel == "fused_region", "descriptor round trip");
  }
  EXPECT(!loadArtifactFromRoot(g_tmp + "/no_such_root"), "missing artifact root");
  EXPECT(!parseDescriptor("ELF..."), "foreign binary rejected");

  // run manifest
  std::ofstream(g_tmp + "/m.json") << R"({"task_id":"main","backend":"sim","artifact_root":")" << g_tmp
                                   << R"(/art","inputs":[{"name":"a","path":"a.npy"},{"name":"b","path":"b.npy","shape":[4,4],"dtype":"f32"}],
      "outputs":[{"name":"out","path":"o.npy"}],"expected_outputs":[{"name":"out","path":"e.npy"}],
      "tiling":{"schema":"s.json","params":"dim_arg0_0=4,dim_arg0_1=4"},
      "block_dim":40,"workspace_size":16777216,"profiling":true,"atol":10,"rtol":1e-2})";
  auto m = loadRunManifest(g_tmp + "/m.json");
  EXPECT((bool)m, "run manifest parses");
  if (m) {
    const auto &t = m->tasks[0];
    EXPECT(m->backend == "sim" && m->tasks.size() == 1 && t.taskId == "main", "task id / backend");
    EXPECT(t.invocation.inputs.size() == 2 && t.invocation.inputs[1].shape == (std::vector<int64_t>{4, 4}) &&
               t.invocation.inputs[1].dtype && *t.invocation.inputs[1].dtype == DType::F32, "input bindings");
    EXPECT(t.invocation.blockDim == 40 && t.invocation.workspaceSize == 16777216 && t.invocation.enableProfiling &&
               t.invocation.atol == 10.0 && t.invocation.rtol == 1e-2, "invocation settings");
    EXPECT(t.invocation.tiling && t.invocation.tiling->params == "dim_arg0_0=4,dim_arg0_1=4", "tiling binding");
  }
  std::ofstream(g_tmp + "/d.json") << R"({"task_id":"main","backend":"hip","artifact_root":"x"})";
  auto d = loadRunManifest(g_tmp + "/d.json");
  EXPECT((bool)d && d->tasks[0].invocation.blockDim == 1 && d->tasks[0].invocation.workspaceSize == 8192 &&
             d->tasks[0].invocation.atol == 1.0 && d->tasks[0].invocation.rtol == 1e-2,
         "defaults: blockDim 1, workspace 8192, atol 1.0, rtol 1e-2");
  std::ofstream(g_tmp + "/nb.json") << R"({"task_id":"main","artifact_root":"x"})";
  EXPECT(!loadRunManifest(g_tmp + "/nb.json"), "backend is required");
  std::ofstream(g_tmp + "/nr.json") << R"({"task_id":"main","backend":"hip"})";
  EXPECT(!loadRunManifest(g_tmp + "/nr.json"), "artifact_root is required");
  std::ofstream(g_tmp + "/bb.json") << R"({"task_id":"main","backend":"tpu","artifact_root":"x"})";
  EXPECT(!loadRunManifest(g_tmp + "/bb.json"), "unknown backend rejected");
  std::ofstream(g_tmp + "/tasks.json") << R"({"backend":"hip","artifact_root":"x","tasks":[{"task_id":"a"},{"task_id":"b","dependencies":["a"]}]})";
  auto tk = loadRunManifest(g_tmp + "/tasks.json");
  EXPECT((bool)tk && tk->tasks.size() == 2 && tk->tasks[1].dependencies.size() == 1 && tk->tasks[1].artifactRoot == "x",
         "tasks array with default artifact root");
}

// Task ordering (reference: lib/Runtime/Execution/TaskGraph.cpp:33-79 and its
// tests in test/tools/runtime/test_taskgraph_runtime.cpp): dependencies first,
// ready tasks in manifest order, unknown / duplicate / cyclic graphs rejected.
static void testPlan() {
  auto task = [](const char *id, std::vector<std::string> deps) {
    RunTaskSpec t;
    t.taskId = id;
    t.dependencies = std::move(deps);
    return t;
  };
  RunManifestSpec m;
  m.tasks = {task("d", {"b", "c"}), task("b", {"a"}), task("c", {"a"}), task("a", {}), task("e", {})};
  auto order = planTasks(m);
  EXPECT((bool)order, "diamond plans");
  if (order) {
    std::string ids;
    for (size_t i : *order) ids += m.tasks[i].taskId;
    EXPECT(ids == "aebcd", "ready tasks in manifest order, dependencies first");
  }
  m.tasks = {task("a", {"zz"})};
  EXPECT(!planTasks(m) && planTasks(m).error() == "unknown task dependency", "unknown dependency");
  m.tasks = {task("a", {}), task("a", {})};
  EXPECT(!planTasks(m) && planTasks(m).error() == "duplicate task id", "duplicate id");
  m.tasks = {task("a", {"b"}), task("b", {"a"})};
  EXPECT(!planTasks(m) && planTasks(m).error() == "task graph contains a cycle", "cycle");
  m.tasks = {task("", {})};
  EXPECT(!planTasks(m) && planTasks(m).error() == "empty task id", "empty id");
}

int main(int argc, char **argv) {
  if (argc < 2) {
    std::printf("usage: %s <tmpdir>\n", argv[0]);
    return 2;
  }
  g_tmp = argv[1];
  testNpy();
  testTiling();
  testComparator();
  testArtifactsAndManifests();
  testPlan();
  std::printf("%d passed, %d failed\n", g_pass, g_fail);
  return g_fail ? 1 : 0;
}
