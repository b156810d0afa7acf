// C ABI of libafir_hip_kernels.so: launcher symbols in the reference's
// dynamic-library-artifact shape, a kernel registry and name-based dispatch.
// Declarations and the reference interfaces they stand in for are in
// include/afir_hip_kernels.h.
#include "afir_hip_kernels.h"

#include <cstdio>
#include <cstring>
#include <string>

#include "../kernels/kernels.h"

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

}  // namespace

extern "C" {

const char *afir_hip_last_error(void) { return g_last_error.c_str(); }

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
  const uint32_t bits = (uint32_t)((uint64_t)f[3] & 0xffffffffu);
  float alpha;
  std::memcpy(&alpha, &bits, 4);
  return finish(afir::launch_matmul_add_leakyrelu(
      static_cast<const uint16_t *>(a), static_cast<const uint16_t *>(b),
      static_cast<const uint16_t *>(bias), static_cast<uint16_t *>(out), f[0], f[1], f[2], alpha,
      block_dim, static_cast<hipStream_t>(stream)));
}

uint32_t afir_hip_probe_mfma_rate(void *stream, const void *operands, void *sink, uint32_t iters,
                                  uint64_t *flops) {
  return finish(afir::launch_mfma_rate_probe(operands, static_cast<float *>(sink), iters, flops,
                                             static_cast<hipStream_t>(stream)));
}

int afir_hip_kernel_count(void) { return kNumKernels; }

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
