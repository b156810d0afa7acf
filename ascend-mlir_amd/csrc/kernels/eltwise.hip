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

// The same chain with the chip's reads and writes separated in time (common.h: HBM serves a
// read phase and a write phase faster than their mixture).  Every lane of the launch is resident
// at once (2048 lanes per CU, 54 registers) and keeps its eight result chunks in registers: it
// reads a and b in kPhasedRounds rounds of kPhasedPer chunks each (all 16 loads at once do not fit
// 64 registers beside the results), computes as the rounds arrive, and holds its stores back
// until the chip's reads have been served.  [4096, 4096]: 31.8 -> 30.4 us (0.79 -> 0.826 of the
// HBM peak) with two rounds of four chunks; four rounds of two measured 0.80.
#ifndef AFIR_ELTWISE_PHASED
#define AFIR_ELTWISE_PHASED 1
#endif
#ifndef AFIR_ELTWISE_PHASE_GBS
#define AFIR_ELTWISE_PHASE_GBS 6700
#endif
#ifndef AFIR_ELTWISE_PHASE_BASE_NS
#define AFIR_ELTWISE_PHASE_BASE_NS 300
#endif
#ifndef AFIR_PHASE_ESTIMATE
#define AFIR_PHASE_ESTIMATE 100
#endif
// smaller launches take the other kernel
#ifndef AFIR_ELTWISE_PHASED_MIN_WG_PER_CU
#define AFIR_ELTWISE_PHASED_MIN_WG_PER_CU 2
#endif
#ifndef AFIR_ELTWISE_PHASED_ROUNDS
#define AFIR_ELTWISE_PHASED_ROUNDS 2
#endif
constexpr int kPhasedRounds = AFIR_ELTWISE_PHASED_ROUNDS, kPhasedPer = 8 / kPhasedRounds;
constexpr int kPhasedChunksPerBlock = kThreads * kPhasedRounds * kPhasedPer;
constexpr int kPhasedLanesPerCU = 2048;
__global__ __launch_bounds__(kThreads, 8) void add_mul_f32_phased(const f32x4 *__restrict__ a,
                                                                  const f32x4 *__restrict__ b,
                                                                  f32x4 *__restrict__ out, int hold_ticks) {
  const long long t_start = wall_clock64();
  // a base per chunk that is the same for the whole workgroup (scalar registers) plus one 32-bit
  // offset per lane: no address registers beside the data
  const size_t block = (size_t)blockIdx.x * kPhasedChunksPerBlock;
  const char *pa = reinterpret_cast<const char *>(a + block), *pb = reinterpret_cast<const char *>(b + block);
  char *po = reinterpret_cast<char *>(out + block);
  const uint32_t lane = threadIdx.x * 16u;
  auto at = [&](const char *p, int k) { return reinterpret_cast<const f32x4 *>(p + (size_t)k * kThreads * 16 + lane); };
  f32x4 r[kPhasedRounds][kPhasedPer];
#pragma unroll
  for (int q = 0; q < kPhasedRounds; ++q) {
    f32x4 x[kPhasedPer], y[kPhasedPer];
#pragma unroll
    for (int u = 0; u < kPhasedPer; ++u) {
      x[u] = load_nt(at(pa, q * kPhasedPer + u));
      y[u] = load_nt(at(pb, q * kPhasedPer + u));
    }
#pragma unroll
    for (int u = 0; u < kPhasedPer; ++u) r[q][u] = (x[u] + y[u]) * y[u];
    // (the next round's loads stay behind this round's results: issued earlier they would take
    // registers the results need)
    __builtin_amdgcn_sched_barrier(0);
  }
  // (the asm makes the results exist here, so the wait for the last loads sits before the hold)
#pragma unroll
  for (int q = 0; q < kPhasedRounds; ++q)
#pragma unroll
    for (int u = 0; u < kPhasedPer; ++u) asm volatile("" : "+v"(r[q][u]));
#if AFIR_PHASE_ESTIMATE
  hold_ticks = phase_hold_here(hold_ticks, t_start, AFIR_PHASE_ESTIMATE * 0.01f);
#endif
  for (int spin = 0; spin < kPhaseSpinLimit && wall_clock64() - t_start < hold_ticks; ++spin)
    __builtin_amdgcn_s_sleep(1);
#pragma unroll
  for (int q = 0; q < kPhasedRounds; ++q)
#pragma unroll
    for (int u = 0; u < kPhasedPer; ++u)
      store_nt(reinterpret_cast<f32x4 *>(po + (size_t)(q * kPhasedPer + u) * kThreads * 16 + lane), r[q][u]);
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
  size_t n4 = vec ? n / 4 : 0;
  size_t done4 = 0;   // chunks the phased kernel has taken
  // whole blocks of a launch of up to twice the chip's resident lanes: the phased kernel
  // (kPhaseMaxLaunches); what is left over: below
  const size_t phased_blocks = n4 / kPhasedChunksPerBlock;
  static const int fit = resident_blocks_per_cu(add_mul_f32_phased, kThreads, 0);   // workgroups per compute unit
  const size_t capacity = fit >= kPhasedLanesPerCU / kThreads ? (size_t)device_cus() * kPhasedLanesPerCU / kThreads : 0;   // blocks per launch
  const int base_ns = env_int("AFIR_ELTWISE_PHASE_BASE_NS", AFIR_ELTWISE_PHASE_BASE_NS, 0, 100000);
  const int gbs = env_int("AFIR_ELTWISE_PHASE_GBS", AFIR_ELTWISE_PHASE_GBS, 100, 100000);
  if (AFIR_ELTWISE_PHASED && !block_dim && capacity > 0 && phased_blocks >= (size_t)device_cus() * AFIR_ELTWISE_PHASED_MIN_WG_PER_CU &&
      phased_blocks <= kPhaseMaxLaunches * capacity && phased_enabled()) {
    const size_t launches = (phased_blocks + capacity - 1) / capacity;
    const size_t take = (phased_blocks + launches - 1) / launches;
    for (size_t b0 = 0; b0 < phased_blocks; b0 += take) {
      const size_t nblocks = phased_blocks - b0 < take ? phased_blocks - b0 : take;
      const int hold_ticks = phase_hold_ticks((int64_t)(nblocks * kPhasedChunksPerBlock * 32), base_ns, gbs);
      AFIR_LAUNCH("add_mul_f32_phased", add_mul_f32_phased, dim3((unsigned)nblocks), dim3(kThreads), 0, stream,
                         reinterpret_cast<const f32x4 *>(a) + b0 * kPhasedChunksPerBlock,
                         reinterpret_cast<const f32x4 *>(b) + b0 * kPhasedChunksPerBlock,
                         reinterpret_cast<f32x4 *>(out) + b0 * kPhasedChunksPerBlock, hold_ticks);
    }
    done4 = phased_blocks * kPhasedChunksPerBlock;
  }
  if (n4 > done4) {
    const size_t rest4 = n4 - done4;
    size_t blocks = (rest4 + (size_t)kThreads * kUnroll - 1) / ((size_t)kThreads * kUnroll);
    if (block_dim) blocks = block_dim;
    if (blocks > 0x7fffffffu) blocks = 0x7fffffffu;
    AFIR_LAUNCH("add_mul_f32_vec", add_mul_f32_vec, dim3((unsigned)blocks), dim3(kThreads), 0, stream,
                       reinterpret_cast<const f32x4 *>(a) + done4, reinterpret_cast<const f32x4 *>(b) + done4,
                       reinterpret_cast<f32x4 *>(out) + done4, rest4);
  }
  if (n4 * 4 < n) {
    size_t rest = n - n4 * 4;
    size_t blocks = (rest + kThreads - 1) / kThreads;
    if (blocks > (size_t)device_cus() * AFIR_ELTWISE_WG_PER_CU) blocks = (size_t)device_cus() * AFIR_ELTWISE_WG_PER_CU;
    if (block_dim && blocks > block_dim) blocks = block_dim;
    AFIR_LAUNCH("add_mul_f32_scalar", add_mul_f32_scalar, dim3((unsigned)blocks), dim3(kThreads), 0, stream,
                       a, b, out, n4 * 4, n);
  }
  return after_launch();
}

}  // namespace afir
