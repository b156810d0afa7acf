// Host-side entry points of the gfx950 fused kernels (C++ level).  The C ABI
// in include/afir_hip_kernels.h is a thin layer over these.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "common.h"

namespace afir {

// out = (a + b) * b, f32, n = rows * cols elements.
LaunchStatus launch_fused_add_mul(const float *a, const float *b, float *out,
                                  int64_t rows, int64_t cols, uint32_t block_dim,
                                  hipStream_t stream);

// y[i] = sum_j (x[i,j] + bias[j]), f32.
LaunchStatus launch_broadcast_add_reducesum(const float *x, const float *bias, float *y,
                                            int64_t m, int64_t n, uint32_t block_dim,
                                            hipStream_t stream);

// out[b,j,i] = f16(relu(x[b,i,j]) + c[j]).
LaunchStatus launch_relu_broadcast_add_transpose(const uint16_t *x, const uint16_t *c,
                                                 uint16_t *out, int64_t nb, int64_t m,
                                                 int64_t n, uint32_t block_dim,
                                                 hipStream_t stream);

// out[r,:] = f16(table[idx[r],:] * scale + shift).
LaunchStatus launch_gather_scale_shift(const uint16_t *table, const int32_t *idx,
                                       const uint16_t *scale, const uint16_t *shift,
                                       uint16_t *out, int32_t *error_flag, int64_t rows,
                                       int64_t dim, int64_t nidx, uint32_t block_dim,
                                       hipStream_t stream);

// out = bf16(max(v, v*alpha)), or bf16(max(v, 0)) with relu set; v = A@B + bias, f32 accumulate.
LaunchStatus launch_matmul_add_leakyrelu(const uint16_t *a, const uint16_t *b,
                                         const uint16_t *bias, uint16_t *out, int64_t m,
                                         int64_t k, int64_t n, float alpha, bool relu,
                                         uint32_t block_dim, hipStream_t stream);

// The same with f16 A, B and f32 bias, out (the types of the reference's matmul
// example, examples/matmul-add-leakyrelu/step0_input.mlir:10-15).
LaunchStatus launch_matmul_add_leakyrelu_f16(const uint16_t *a, const uint16_t *b, const float *bias,
                                             float *out, int64_t m, int64_t k, int64_t n,
                                             float alpha, bool relu, uint32_t block_dim,
                                             hipStream_t stream);

// Matmul with transposed and / or batched operands (matmul_layouts.hip): A as [M, K] or, with
// trans_a, [K, M]; B as [K, N] or, with trans_b, [N, K]; `batch` independent products of
// densely packed matrices; bias [N] (null: none) shared by the batches.  f16io selects f16 A, B
// with float32 bias and out; otherwise everything is bf16.  Plain, unbatched calls go to the
// kernels above.
LaunchStatus launch_matmul_layouts(const uint16_t *a, const uint16_t *b, const void *bias, void *out, bool f16io,
                                   int64_t batch, int64_t m, int64_t k, int64_t n, bool trans_a, bool trans_b,
                                   float alpha, bool relu, uint32_t block_dim, hipStream_t stream);

// Fast path of the matmul for tile-aligned shapes (matmul_dma.hip).
bool matmul_dma_supported(int64_t m, int64_t k, int64_t n);
LaunchStatus launch_matmul_dma(const uint16_t *a, const uint16_t *b, const uint16_t *bias,
                               uint16_t *out, int m, int k, int n, float alpha, bool relu,
                               uint32_t block_dim, hipStream_t stream);
LaunchStatus launch_matmul_dma_f16(const uint16_t *a, const uint16_t *b, const float *bias,
                                   float *out, int m, int k, int n, float alpha, bool relu,
                                   uint32_t block_dim, hipStream_t stream);
// `batch` products of one shape, A [batch, m, k], B [batch, k, n], out [batch, m, n] densely
// packed, the bias [n] shared (null: none); shapes as matmul_dma_supported(m, k, n) says
LaunchStatus launch_matmul_dma_batched(const uint16_t *a, const uint16_t *b, const void *bias, void *out, bool f16io,
                                       int batch, int m, int k, int n, float alpha, bool relu, hipStream_t stream);

inline LaunchStatus ok_status() { return LaunchStatus{0u, ""}; }
inline LaunchStatus invalid(const char *msg) { return LaunchStatus{1u, msg}; }
inline LaunchStatus after_launch() {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return LaunchStatus{2u, hipGetErrorString(e)};
  return ok_status();
}

}  // namespace afir
