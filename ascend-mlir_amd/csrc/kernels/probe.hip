// Measurement aid: the rate at which the matrix cores retire
// v_mfma_f32_32x32x16_bf16 when nothing else happens -- operands and
// accumulators live in registers, the loop touches no memory.  The result
// depends on the operand VALUES: the chip runs against a board power limit,
// and operands with random mantissas toggle far more logic per instruction
// than constant ones, so the sustained clock (and with it the attainable
// fraction of the published peak) differs between the two.  The benchmark
// reports this rate for the workload's own operand distribution next to the
// matmul kernel's figure.
#include "kernels.h"

namespace afir {

namespace {

constexpr int kProbeThreads = 512;   // 8 waves, two per SIMD
constexpr int kProbeAcc = 8;         // independent accumulators per wave
constexpr int kProbeOps = 4;         // operand register pairs cycled through

__global__ __launch_bounds__(kProbeThreads) void mfma_rate_probe(const u32x4 *__restrict__ operands,
                                                                 float *__restrict__ sink,
                                                                 int iters) {
  f32x16 acc[kProbeAcc];
#pragma unroll
  for (int i = 0; i < kProbeAcc; ++i)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[i][e] = 0.f;
  bf16x8 a[kProbeOps], b[kProbeOps];
#pragma unroll
  for (int o = 0; o < kProbeOps; ++o) {
    a[o] = __builtin_bit_cast(bf16x8, operands[(threadIdx.x * kProbeOps + o) * 2]);
    b[o] = __builtin_bit_cast(bf16x8, operands[(threadIdx.x * kProbeOps + o) * 2 + 1]);
  }
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int o = 0; o < kProbeOps; ++o)
#pragma unroll
      for (int i = 0; i < kProbeAcc; ++i)
        acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[o], b[(o + i) % kProbeOps], acc[i], 0,
                                                         0, 0);
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < kProbeAcc; ++i)
#pragma unroll
    for (int e = 0; e < 16; ++e) s += acc[i][e];
  sink[(size_t)blockIdx.x * kProbeThreads + threadIdx.x] = s;
}

}  // namespace

LaunchStatus launch_mfma_rate_probe(const void *operands, float *sink, uint32_t iters,
                                    uint64_t *flops, hipStream_t stream) {
  if (!operands || !sink) return invalid("mfma_rate_probe: null pointer");
  if (!aligned16(operands)) return invalid("mfma_rate_probe: operands must be 16-byte aligned");
  if (iters == 0 || iters > (1u << 24)) return invalid("mfma_rate_probe: iters out of range");
  const unsigned blocks = 2u * kNumCU;
  hipLaunchKernelGGL(mfma_rate_probe, dim3(blocks), dim3(kProbeThreads), 0, stream,
                     static_cast<const u32x4 *>(operands), sink, (int)iters);
  if (flops)
    *flops = 2ull * 32 * 32 * 16 * kProbeAcc * kProbeOps * (uint64_t)iters *
             (kProbeThreads / kWave) * blocks;
  return after_launch();
}

}  // namespace afir
