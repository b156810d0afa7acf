// Measurement aids of the benchmark (declared in probes.h).
//
// mfma_rate_probe: the rate at which the matrix cores retire
// v_mfma_f32_16x16x32_bf16 -- the instruction of the matmul kernel -- when
// nothing else happens: operands and accumulators live in registers, the loop
// touches no memory.  The result depends on the operand VALUES: the chip runs
// against a board power limit, and operands with random mantissas toggle far
// more logic per instruction than constant ones, so the sustained clock (and
// with it the attainable fraction of the published peak) differs between the
// two.  (The 32x32x16 form of the instruction sustains 15 % less on random
// operands, 1765 against 2040 TFLOP/s, and the same 2470 on constant ones.)
#include "probes.h"

#include "../kernels/kernels.h"
#include "matmul_feed_probes.h"

namespace afir {

constexpr int kProbeThreads = 512;   // 8 waves, two per SIMD
constexpr int kProbeAcc = 16;        // independent accumulators per wave
constexpr int kProbeOps = 4;         // operand register pairs cycled through

__global__ __launch_bounds__(kProbeThreads) void mfma_rate_probe(const u32x4 *__restrict__ operands,
                                                                 float *__restrict__ sink,
                                                                 int iters) {
  f32x4 acc[kProbeAcc];
#pragma unroll
  for (int i = 0; i < kProbeAcc; ++i)
#pragma unroll
    for (int e = 0; e < 4; ++e) acc[i][e] = 0.f;
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
        acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[o], b[(o + i) % kProbeOps], acc[i], 0, 0, 0);
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < kProbeAcc; ++i)
#pragma unroll
    for (int e = 0; e < 4; ++e) s += acc[i][e];
  sink[(size_t)blockIdx.x * kProbeThreads + threadIdx.x] = s;
}

}  // namespace afir

namespace {

using afir::kNumCU;
using afir::u32x4;
using afir::f32x4;

constexpr int kCopyThreads = 256, kCopyUnroll = 4;

__global__ __launch_bounds__(kCopyThreads) void probe_copy(const u32x4 *__restrict__ src, u32x4 *__restrict__ dst,
                                                           size_t n16) {
  const size_t chunk = (size_t)kCopyThreads * kCopyUnroll, stride = (size_t)gridDim.x * chunk;
  for (size_t base = (size_t)blockIdx.x * chunk; base < n16; base += stride) {
    u32x4 v[kCopyUnroll];
#pragma unroll
    for (int u = 0; u < kCopyUnroll; ++u) v[u] = afir::load_nt(src + base + u * kCopyThreads + threadIdx.x);
#pragma unroll
    for (int u = 0; u < kCopyUnroll; ++u) afir::store_nt(dst + base + u * kCopyThreads + threadIdx.x, v[u]);
  }
}

__global__ __launch_bounds__(kCopyThreads) void probe_read(const f32x4 *__restrict__ src, float *__restrict__ sink,
                                                           size_t n16) {
  __shared__ float part[kCopyThreads / 64];
  const size_t chunk = (size_t)kCopyThreads * kCopyUnroll, stride = (size_t)gridDim.x * chunk;
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  for (size_t base = (size_t)blockIdx.x * chunk; base < n16; base += stride) {
    f32x4 v[kCopyUnroll];
#pragma unroll
    for (int u = 0; u < kCopyUnroll; ++u) v[u] = afir::load_nt(src + base + u * kCopyThreads + threadIdx.x);
#pragma unroll
    for (int u = 0; u < kCopyUnroll; ++u) acc += v[u];
  }
  const float s = afir::wave_sum((acc.x + acc.y) + (acc.z + acc.w));
  if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = s;
  __syncthreads();
  if (threadIdx.x == 0) sink[blockIdx.x] = (part[0] + part[1]) + (part[2] + part[3]);
}

// one 64 x 64 tile of 2-byte elements per workgroup, tiles numbered along m first
__global__ __launch_bounds__(kCopyThreads) void probe_tilecopy64(const uint16_t *__restrict__ x,
                                                                 uint16_t *__restrict__ out, int nb, int m, int n) {
  const int t = threadIdx.x;
  const unsigned tiles_m = (unsigned)(m / 64), tiles_n = (unsigned)(n / 64);
  const unsigned ntiles = (unsigned)nb * tiles_m * tiles_n;
  const int chunk = (t & 7) * 8, row = t >> 3;
  for (unsigned tile_id = blockIdx.x; tile_id < ntiles; tile_id += gridDim.x) {
    const unsigned rest = tile_id / tiles_m;
    const int tm = (int)(tile_id - rest * tiles_m);
    const int b = (int)(rest / tiles_n);
    const int tn = (int)(rest - (unsigned)b * tiles_n);
    const int m0 = tm * 64, n0 = tn * 64;
    u32x4 v[2];
#pragma unroll
    for (int k = 0; k < 2; ++k)
      v[k] = *reinterpret_cast<const u32x4 *>(x + ((int64_t)b * m + m0 + row + 32 * k) * n + n0 + chunk);
#pragma unroll
    for (int k = 0; k < 2; ++k)
      afir::store_nt(reinterpret_cast<u32x4 *>(out + ((int64_t)b * n + n0 + row + 32 * k) * m + m0 + chunk), v[k]);
  }
}

// write-only stream: every lane stores a value of its own
__global__ __launch_bounds__(kCopyThreads) void probe_fill(u32x4 *__restrict__ dst, size_t n16, uint32_t seed) {
  const size_t chunk = (size_t)kCopyThreads * kCopyUnroll, stride = (size_t)gridDim.x * chunk;
  const u32x4 v = {seed, threadIdx.x, blockIdx.x, seed * 3u};
  for (size_t base = (size_t)blockIdx.x * chunk; base < n16; base += stride) {
#pragma unroll
    for (int u = 0; u < kCopyUnroll; ++u) afir::store_nt(dst + base + u * kCopyThreads + threadIdx.x, v);
  }
}

// the copy with every lane resident at once (eight 16-byte chunks per lane) and the stores held
// back until `hold_ticks` of the real-time counter after the workgroup's start
constexpr int kPhasedChunks = 8;
__global__ __launch_bounds__(kCopyThreads, 8) void probe_copy_phased(const u32x4 *__restrict__ src,
                                                                     u32x4 *__restrict__ dst, int hold_ticks) {
  const long long t_start = wall_clock64();
  const size_t base = (size_t)blockIdx.x * (kCopyThreads * kPhasedChunks) + threadIdx.x;
  u32x4 v[kPhasedChunks];
#pragma unroll
  for (int u = 0; u < kPhasedChunks; ++u) v[u] = afir::load_nt(src + base + u * kCopyThreads);
#pragma unroll
  for (int u = 0; u < kPhasedChunks; ++u) asm volatile("" : "+v"(v[u]));
  for (int spin = 0; spin < afir::kPhaseSpinLimit && wall_clock64() - t_start < hold_ticks; ++spin)
    __builtin_amdgcn_s_sleep(1);
#pragma unroll
  for (int u = 0; u < kPhasedChunks; ++u) afir::store_nt(dst + base + u * kCopyThreads, v[u]);
}

uint32_t done() { return hipGetLastError() == hipSuccess ? 0u : 2u; }

}  // namespace

extern "C" {

uint32_t afir_bench_mfma_rate(void *stream, const void *operands, void *sink, uint32_t iters, uint64_t *flops) {
  if (!operands || !sink || !afir::aligned16(operands)) return 1u;
  if (iters == 0 || iters > (1u << 24)) return 1u;
  const unsigned blocks = 2u * kNumCU;
  hipLaunchKernelGGL(afir::mfma_rate_probe, dim3(blocks), dim3(afir::kProbeThreads), 0,
                     static_cast<hipStream_t>(stream), static_cast<const u32x4 *>(operands),
                     static_cast<float *>(sink), (int)iters);
  if (flops)
    *flops = 2ull * 16 * 16 * 32 * afir::kProbeAcc * afir::kProbeOps * (uint64_t)iters *
             (afir::kProbeThreads / afir::kWave) * blocks;
  return done();
}

uint32_t afir_bench_matmul_ablated(void *stream, const void *a, const void *b, const void *bias, void *out, int m,
                                   int k, int n, int what) {
  namespace dma = afir::dma;
  if (!a || !b || !bias || !out || (what < 1 || what > 4) || !dma::supported(m, k, n)) return 1u;
  const uint16_t *pa = static_cast<const uint16_t *>(a), *pb = static_cast<const uint16_t *>(b);
  hipStream_t st = static_cast<hipStream_t>(stream);
  switch (what) {
    case 1: return dma::launch<false, dma::NoLoads>("matmul_dma_no_loads", pa, pb, bias, out, m, k, n, 0.01f, false, 0, st).code;
    case 2: return dma::launch<false, dma::NoLoadsNoReads>("matmul_dma_no_loads_no_reads", pa, pb, bias, out, m, k, n, 0.01f, false, 0, st).code;
    case 3: return dma::launch<false, dma::LoadsOfOneKiB>("matmul_dma_loads_of_one_kib", pa, pb, bias, out, m, k, n, 0.01f, false, 0, st).code;
    default: return dma::launch<false, dma::L2Resident>("matmul_dma_l2_resident", pa, pb, bias, out, m, k, n, 0.01f, false, 0, st).code;
  }
}

uint32_t afir_bench_copy(void *stream, const void *src, void *dst, size_t bytes) {
  if (!src || !dst || bytes == 0 || bytes % 16384 != 0 || !afir::aligned16(src) || !afir::aligned16(dst)) return 1u;
  hipLaunchKernelGGL(probe_copy, dim3(4u * kNumCU), dim3(kCopyThreads), 0, static_cast<hipStream_t>(stream),
                     static_cast<const u32x4 *>(src), static_cast<u32x4 *>(dst), bytes / 16);
  return done();
}

uint32_t afir_bench_fill(void *stream, void *dst, size_t bytes, uint32_t seed) {
  if (!dst || bytes == 0 || bytes % 16384 != 0 || !afir::aligned16(dst)) return 1u;
  hipLaunchKernelGGL(probe_fill, dim3(8u * kNumCU), dim3(kCopyThreads), 0, static_cast<hipStream_t>(stream),
                     static_cast<u32x4 *>(dst), bytes / 16, seed);
  return done();
}

uint32_t afir_bench_copy_phased(void *stream, const void *src, void *dst, size_t bytes) {
  const size_t per_block = (size_t)kCopyThreads * kPhasedChunks * 16;
  if (!src || !dst || bytes == 0 || bytes % per_block != 0 || !afir::aligned16(src) || !afir::aligned16(dst)) return 1u;
  // (every lane resident at once: 2048 lanes per CU)
  if (bytes / per_block * kCopyThreads > (size_t)afir::device_cus() * 2048) return 1u;
  const int hold_ticks = afir::phase_hold_ticks((int64_t)bytes, 300, 6700);
  hipLaunchKernelGGL(probe_copy_phased, dim3((unsigned)(bytes / per_block)), dim3(kCopyThreads), 0,
                     static_cast<hipStream_t>(stream), static_cast<const u32x4 *>(src), static_cast<u32x4 *>(dst),
                     hold_ticks);
  return done();
}

uint32_t afir_bench_read(void *stream, const void *src, void *sink, size_t bytes) {
  if (!src || !sink || bytes == 0 || bytes % 16384 != 0 || !afir::aligned16(src)) return 1u;
  hipLaunchKernelGGL(probe_read, dim3(8u * kNumCU), dim3(kCopyThreads), 0, static_cast<hipStream_t>(stream),
                     static_cast<const f32x4 *>(src), static_cast<float *>(sink), bytes / 16);
  return done();
}

uint32_t afir_bench_tilecopy64(void *stream, const void *x, void *out, int nb, int m, int n) {
  if (!x || !out || nb <= 0 || m <= 0 || n <= 0 || m % 64 || n % 64 || !afir::aligned16(x) || !afir::aligned16(out))
    return 1u;
  const int64_t tiles = (int64_t)nb * (m / 64) * (n / 64);
  if (tiles >= ((int64_t)1 << 31)) return 1u;
  hipLaunchKernelGGL(probe_tilecopy64, dim3((unsigned)tiles), dim3(kCopyThreads), 0, static_cast<hipStream_t>(stream),
                     static_cast<const uint16_t *>(x), static_cast<uint16_t *>(out), nb, m, n);
  return done();
}

}  // extern "C"
