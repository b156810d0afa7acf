// Fused elementwise chain out = (a + b) * b for f32 (afir.add -> afir.mul,
// reference lowering lib/Conversion/AFIRToASCIR/Math/Elementwise.cpp:25-57).
//
// HBM-bound: 12 algorithmic bytes per element (two reads, one write).  Each
// lane moves 128 bits per access; a workgroup issues kUnroll independent
// loads per input before the first use so a wave keeps 2*kUnroll KiB in
// flight.  Loads and stores are non-temporal: every byte is touched once.
// The add and the mul stay two IEEE operations (no contraction is possible
// in (a+b)*b), which keeps the result bit-identical to the CPU golden.
#include "kernels.h"

namespace afir {

namespace {

constexpr int kThreads = 256;
#ifndef AFIR_ELTWISE_UNROLL
#define AFIR_ELTWISE_UNROLL 2   // 128-bit loads per input in flight per lane (2, 4, 8 measured within 3 %)
#endif
#ifndef AFIR_ELTWISE_WG_PER_CU
#define AFIR_ELTWISE_WG_PER_CU 16
#endif
constexpr int kUnroll = AFIR_ELTWISE_UNROLL;

__global__ __launch_bounds__(kThreads) void add_mul_f32_vec(const f32x4 *__restrict__ a,
                                                            const f32x4 *__restrict__ b,
                                                            f32x4 *__restrict__ out,
                                                            size_t n4) {
  const size_t chunk = (size_t)kThreads * kUnroll;
  const size_t stride = (size_t)gridDim.x * chunk;
  for (size_t base = (size_t)blockIdx.x * chunk; base < n4; base += stride) {
    f32x4 va[kUnroll], vb[kUnroll];
    if (base + chunk <= n4) {
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        size_t i = base + (size_t)u * kThreads + threadIdx.x;
        va[u] = load_nt(a + i);
        vb[u] = load_nt(b + i);
      }
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        size_t i = base + (size_t)u * kThreads + threadIdx.x;
        store_nt(out + i, (va[u] + vb[u]) * vb[u]);
      }
    } else {
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        size_t i = base + (size_t)u * kThreads + threadIdx.x;
        if (i < n4) {
          f32x4 x = load_nt(a + i), y = load_nt(b + i);
          store_nt(out + i, (x + y) * y);
        }
      }
    }
  }
}

// Tail elements and unaligned buffers.
__global__ __launch_bounds__(kThreads) void add_mul_f32_scalar(const float *__restrict__ a,
                                                               const float *__restrict__ b,
                                                               float *__restrict__ out,
                                                               size_t begin, size_t n) {
  size_t stride = (size_t)gridDim.x * kThreads;
  for (size_t i = begin + (size_t)blockIdx.x * kThreads + threadIdx.x; i < n; i += stride) {
    float y = b[i];
    out[i] = (a[i] + y) * y;
  }
}

}  // namespace

LaunchStatus launch_fused_add_mul(const float *a, const float *b, float *out, int64_t rows,
                                  int64_t cols, uint32_t block_dim, hipStream_t stream) {
  if (rows < 0 || cols < 0) return invalid("fused_add_mul: negative extent");
  if (rows != 0 && cols > INT64_MAX / rows) return invalid("fused_add_mul: extent overflow");
  const size_t n = (size_t)rows * (size_t)cols;
  if (n == 0) return ok_status();
  if (!a || !b || !out) return invalid("fused_add_mul: null tensor pointer");

  const bool vec = aligned16(a) && aligned16(b) && aligned16(out);
  const size_t n4 = vec ? n / 4 : 0;
  if (n4) {
    size_t blocks = (n4 + (size_t)kThreads * kUnroll - 1) / ((size_t)kThreads * kUnroll);
    if (block_dim) blocks = block_dim;
    if (blocks > 0x7fffffffu) blocks = 0x7fffffffu;
    hipLaunchKernelGGL(add_mul_f32_vec, dim3((unsigned)blocks), dim3(kThreads), 0, stream,
                       reinterpret_cast<const f32x4 *>(a), reinterpret_cast<const f32x4 *>(b),
                       reinterpret_cast<f32x4 *>(out), n4);
  }
  if (n4 * 4 < n) {
    size_t rest = n - n4 * 4;
    size_t blocks = (rest + kThreads - 1) / kThreads;
    if (blocks > (size_t)device_cus() * AFIR_ELTWISE_WG_PER_CU) blocks = (size_t)device_cus() * AFIR_ELTWISE_WG_PER_CU;
    if (block_dim && blocks > block_dim) blocks = block_dim;
    hipLaunchKernelGGL(add_mul_f32_scalar, dim3((unsigned)blocks), dim3(kThreads), 0, stream,
                       a, b, out, n4 * 4, n);
  }
  return after_launch();
}

}  // namespace afir
