// Broadcast add + row sum: y[i] = sum_j (x[i,j] + bias[j]), f32
// (reduction generic of lib/Conversion/LinalgToAscendC/ComputeConversion.cpp:246-750;
// golden examples/broadcast-add-reduce/gen_data.py:33 restated with a
// per-column bias).
//
// HBM-bound: x is read once (4 bytes per element), bias stays in cache, one
// float leaves per row.  One wavefront owns a row: lane l reads the 128-bit
// chunks l, l+64, l+128, ... so every load instruction of a wave covers 1 KiB
// of contiguous memory; kUnroll chunks are in flight per lane before the
// first add.  Each lane keeps four running sums (the float4 components), the
// lane total is reduced across the wave with DPP (quad butterflies, row
// mirrors) and the four 16-lane row totals are combined in a fixed order, so
// the result is deterministic.  The broadcast operand is never materialised.
#include <mutex>

#include "afir_hip_kernels.h"
#include "kernels.h"

namespace afir {

namespace {

#ifndef AFIR_ROWSUM_THREADS
#define AFIR_ROWSUM_THREADS 512
#endif
#ifndef AFIR_ROWSUM_UNROLL
#define AFIR_ROWSUM_UNROLL 8
#endif
#ifndef AFIR_ROWSUM_WAVES_PER_CU
#define AFIR_ROWSUM_WAVES_PER_CU 16
#endif
constexpr int kThreads = AFIR_ROWSUM_THREADS;
constexpr int kWavesPerBlock = kThreads / kWave;
constexpr int kUnroll = AFIR_ROWSUM_UNROLL;
constexpr int kWavesPerCU = AFIR_ROWSUM_WAVES_PER_CU;

// Rows of at most 64*CH 128-bit chunks: the wave keeps its CH chunks of bias
// in registers for all the rows it walks.  The row is requested in batches of
// kBatch chunks per lane (a batch is summed while the next is in flight); with
// the default of 16 a row of up to 1024 chunks is one batch, which measured
// faster on MI355X than batches of 2, 4 or 8.  EXACT: the row is exactly 64*CH chunks, no lane is ever idle and
// the loads carry no predicate.
#ifndef AFIR_ROWSUM_BATCH
#define AFIR_ROWSUM_BATCH 16
#endif
template <int CH, bool EXACT>
__global__ __launch_bounds__(kThreads) void bcast_add_rowsum_f32_resident(
    const float *__restrict__ x, const float *__restrict__ bias, float *__restrict__ y,
    int64_t m, int64_t n) {
  constexpr int kBatch = CH < AFIR_ROWSUM_BATCH ? CH : AFIR_ROWSUM_BATCH;
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t wave = (int64_t)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
  const int64_t nwaves = (int64_t)gridDim.x * kWavesPerBlock;
  const int n4 = (int)(n >> 2);
  const f32x4 *b4 = reinterpret_cast<const f32x4 *>(bias);
  const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
  f32x4 vb[CH];
#pragma unroll
  for (int u = 0; u < CH; ++u) vb[u] = (EXACT || lane + u * kWave < n4) ? b4[lane + u * kWave] : zero;

  for (int64_t row = wave; row < m; row += nwaves) {
    const f32x4 *x4 = reinterpret_cast<const f32x4 *>(x + row * n);
    f32x4 acc = zero;
#pragma unroll
    for (int g = 0; g < CH; g += kBatch) {
      f32x4 vx[kBatch];
#pragma unroll
      for (int u = 0; u < kBatch; ++u)
        vx[u] = (EXACT || lane + (g + u) * kWave < n4) ? load_nt(x4 + lane + (g + u) * kWave) : zero;
#pragma unroll
      for (int u = 0; u < kBatch; ++u) acc += vx[u] + vb[g + u];
    }
    float s = (acc.x + acc.y) + (acc.z + acc.w);
    s = wave_sum(s);
    if (lane == 0) y[row] = s;
  }
}

// Rows of exactly 256*U chunks: a workgroup of four waves owns a row, so that
// the grid walks x like a linear stream -- every load instruction of a
// workgroup covers 4 KiB of contiguous memory and the whole grid a window of
// a few MiB -- which this memory system serves ~8 % faster than one wave per
// row.  A lane's U chunks of bias stay in registers.  The next row is
// requested before the current one is reduced (DPP inside the waves, one LDS
// word per wave, one barrier per row: the partial sums are double-buffered by
// row parity).
#ifndef AFIR_ROWSUM_WG_PER_CU
#define AFIR_ROWSUM_WG_PER_CU 2
#endif
constexpr int kRowThreads = 256;
template <int U>
__global__ __launch_bounds__(kRowThreads) void bcast_add_rowsum_f32_wgrow(
    const float *__restrict__ x, const float *__restrict__ bias, float *__restrict__ y,
    int64_t m, int64_t n) {
  __shared__ float part[2][kRowThreads / kWave];
  const int t = threadIdx.x, lane = t & (kWave - 1), wave = t >> 6;
  const f32x4 *b4 = reinterpret_cast<const f32x4 *>(bias);
  f32x4 vb[U], vx[U];
#pragma unroll
  for (int u = 0; u < U; ++u) vb[u] = b4[t + u * kRowThreads];
  int64_t row = blockIdx.x;
  if (row < m) {
    const f32x4 *x4 = reinterpret_cast<const f32x4 *>(x + row * n);
#pragma unroll
    for (int u = 0; u < U; ++u) vx[u] = load_nt(x4 + t + u * kRowThreads);
  }
  int parity = 0;
  for (; row < m; row += gridDim.x) {
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int u = 0; u < U; ++u) acc += vx[u] + vb[u];
    const int64_t next = row + gridDim.x;
    if (next < m) {
      const f32x4 *x4 = reinterpret_cast<const f32x4 *>(x + next * n);
#pragma unroll
      for (int u = 0; u < U; ++u) vx[u] = load_nt(x4 + t + u * kRowThreads);
    }
    float s = (acc.x + acc.y) + (acc.z + acc.w);
    s = wave_sum(s);
    if (lane == 0) part[parity][wave] = s;
    __syncthreads();
    if (t == 0) y[row] = (part[parity][0] + part[parity][1]) + (part[parity][2] + part[parity][3]);
    parity ^= 1;
  }
}

__global__ __launch_bounds__(kThreads) void bcast_add_rowsum_f32_vec(
    const float *__restrict__ x, const float *__restrict__ bias, float *__restrict__ y,
    int64_t m, int64_t n) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t wave = (int64_t)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
  const int64_t nwaves = (int64_t)gridDim.x * kWavesPerBlock;
  const int64_t n4 = n >> 2;
  const f32x4 *b4 = reinterpret_cast<const f32x4 *>(bias);

  for (int64_t row = wave; row < m; row += nwaves) {
    const f32x4 *x4 = reinterpret_cast<const f32x4 *>(x + row * n);
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    int64_t c = lane;
    for (; c + (int64_t)(kUnroll - 1) * kWave < n4; c += (int64_t)kUnroll * kWave) {
      f32x4 vx[kUnroll], vb[kUnroll];
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        vx[u] = load_nt(x4 + c + u * kWave);
        vb[u] = b4[c + u * kWave];
      }
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) acc += vx[u] + vb[u];
    }
    for (; c < n4; c += kWave) acc += load_nt(x4 + c) + b4[c];
    float s = (acc.x + acc.y) + (acc.z + acc.w);
    s = wave_sum(s);
    if (lane == 0) y[row] = s;
  }
}

// Any n, any alignment: one wave per row, scalar accesses.
__global__ __launch_bounds__(kThreads) void bcast_add_rowsum_f32_scalar(
    const float *__restrict__ x, const float *__restrict__ bias, float *__restrict__ y,
    int64_t m, int64_t n) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t wave = (int64_t)blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
  const int64_t nwaves = (int64_t)gridDim.x * kWavesPerBlock;
  for (int64_t row = wave; row < m; row += nwaves) {
    const float *xr = x + row * n;
    float s = 0.f;
    for (int64_t c = lane; c < n; c += kWave) s += xr[c] + bias[c];
    s = wave_sum(s);
    if (lane == 0) y[row] = s;
  }
}

}  // namespace

LaunchStatus launch_broadcast_add_reducesum(const float *x, const float *bias, float *y,
                                            int64_t m, int64_t n, uint32_t block_dim,
                                            hipStream_t stream) {
  if (m < 0 || n < 0) return invalid("broadcast_add_reducesum: negative extent");
  if (m == 0) return ok_status();
  if (!y) return invalid("broadcast_add_reducesum: null output pointer");
  if (n > 0 && (!x || !bias)) return invalid("broadcast_add_reducesum: null input pointer");
  if (n != 0 && m > INT64_MAX / n / 4) return invalid("broadcast_add_reducesum: extent overflow");

  int64_t blocks = (m + kWavesPerBlock - 1) / kWavesPerBlock;
  if (block_dim) blocks = block_dim;
  if (blocks > 0x7fffffff) blocks = 0x7fffffff;
  const bool vec = n > 0 && (n % 4 == 0) && aligned16(x) && aligned16(bias);
  if (vec && (n / 4) % kRowThreads == 0 && n / 4 <= 8 * kRowThreads && aligned16(x) &&
      ((n / 4 / kRowThreads) & (n / 4 / kRowThreads - 1)) == 0) {
    // a workgroup per row
    int64_t wblocks = (int64_t)device_cus() * AFIR_ROWSUM_WG_PER_CU;
    if (wblocks > m) wblocks = m;
    if (block_dim) wblocks = block_dim;
    const dim3 grid((unsigned)wblocks), block(kRowThreads);
    switch ((int)(n / 4 / kRowThreads)) {
      case 1: AFIR_LAUNCH("bcast_add_rowsum_f32_wgrow<1>", bcast_add_rowsum_f32_wgrow<1>, grid, block, 0, stream, x, bias, y, m, n); break;
      case 2: AFIR_LAUNCH("bcast_add_rowsum_f32_wgrow<2>", bcast_add_rowsum_f32_wgrow<2>, grid, block, 0, stream, x, bias, y, m, n); break;
      case 4: AFIR_LAUNCH("bcast_add_rowsum_f32_wgrow<4>", bcast_add_rowsum_f32_wgrow<4>, grid, block, 0, stream, x, bias, y, m, n); break;
      default: AFIR_LAUNCH("bcast_add_rowsum_f32_wgrow<8>", bcast_add_rowsum_f32_wgrow<8>, grid, block, 0, stream, x, bias, y, m, n); break;
    }
  } else if (vec && n / 4 <= 16 * kWave) {
    // persistent waves: each keeps its bias chunks resident and walks several rows
    const int64_t n4 = n / 4;
    int64_t pblocks = (int64_t)device_cus() * kWavesPerCU / kWavesPerBlock;
    if (pblocks * kWavesPerBlock > m) pblocks = (m + kWavesPerBlock - 1) / kWavesPerBlock;
    if (block_dim) pblocks = block_dim;
    const dim3 grid((unsigned)pblocks), block(kThreads);
    auto launch = [&](auto kernel) {
      AFIR_LAUNCH("bcast_add_rowsum_f32_resident", kernel, grid, block, 0, stream, x, bias, y, m, n);
    };
    if (n4 == 16 * kWave) launch(bcast_add_rowsum_f32_resident<16, true>);
    else if (n4 == 8 * kWave) launch(bcast_add_rowsum_f32_resident<8, true>);
    else if (n4 == 4 * kWave) launch(bcast_add_rowsum_f32_resident<4, true>);
    else if (n4 <= 1 * kWave) launch(bcast_add_rowsum_f32_resident<1, false>);
    else if (n4 <= 2 * kWave) launch(bcast_add_rowsum_f32_resident<2, false>);
    else if (n4 <= 4 * kWave) launch(bcast_add_rowsum_f32_resident<4, false>);
    else if (n4 <= 8 * kWave) launch(bcast_add_rowsum_f32_resident<8, false>);
    else launch(bcast_add_rowsum_f32_resident<16, false>);
  } else if (vec) {
    AFIR_LAUNCH("bcast_add_rowsum_f32_vec", bcast_add_rowsum_f32_vec, dim3((unsigned)blocks), dim3(kThreads), 0,
                       stream, x, bias, y, m, n);
  } else {
    AFIR_LAUNCH("bcast_add_rowsum_f32_scalar", bcast_add_rowsum_f32_scalar, dim3((unsigned)blocks), dim3(kThreads), 0,
                       stream, x, bias, y, m, n);
  }
  return after_launch();
}

}  // namespace afir

// ---- the entry point that allocates nothing ---------------------------------
//
// Few, long rows cannot fill the chip with a wavefront or a workgroup per row,
// so the row is cut into chunks of kSplitChunk floats, one workgroup sums one
// chunk (bias included) and leaves a float in a scratch buffer, and a second
// kernel adds a row's partial sums in a fixed order.  The scratch buffer is a
// file-scope device array, so this path needs no allocation and no workspace
// from the caller; every GPU holds its own copy at its own address, looked up
// once per device with hipGetSymbolAddress.  In host code `afir_rowsum_scratch`
// is only the handle for that lookup, never an address to pass to a kernel.
namespace afir {
namespace {

constexpr int kSplitThreads = 256;
constexpr int kSplitUnroll = 8;                                  // 128-bit loads in flight per lane
constexpr int64_t kSplitChunk = (int64_t)kSplitThreads * 4 * kSplitUnroll;   // 8192 floats = 32 KiB
constexpr int64_t kScratchFloats = 65536;                        // 256 KiB per GPU (the array below)

}  // namespace
}  // namespace afir

static __device__ __align__(256) float afir_rowsum_scratch[65536];
static_assert(sizeof(afir_rowsum_scratch) == 65536 * sizeof(float), "the scratch array holds 65536 partial sums");

namespace afir {
namespace {

// partial[row * parts + p] = sum over chunk p of row `row` of (x + bias); the last chunk may be short
__global__ __launch_bounds__(kSplitThreads) void bcast_add_rowsum_f32_split(
    const float *__restrict__ x, const float *__restrict__ bias, float *__restrict__ partial,
    int64_t n, int parts) {
  __shared__ float part[kSplitThreads / kWave];
  const int t = threadIdx.x;
  const int64_t row = blockIdx.x / (unsigned)parts;
  const int p = (int)(blockIdx.x - row * (unsigned)parts);
  const int64_t first = (int64_t)p * kSplitChunk;
  const int64_t n4 = (n - first < kSplitChunk ? n - first : kSplitChunk) >> 2;   // 128-bit chunks here
  const f32x4 *x4 = reinterpret_cast<const f32x4 *>(x + row * n + first);
  const f32x4 *b4 = reinterpret_cast<const f32x4 *>(bias + first);
  const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
  f32x4 vx[kSplitUnroll], vb[kSplitUnroll];
#pragma unroll
  for (int u = 0; u < kSplitUnroll; ++u) {
    const int64_t c = t + (int64_t)u * kSplitThreads;
    vx[u] = c < n4 ? load_nt(x4 + c) : zero;
    vb[u] = c < n4 ? b4[c] : zero;
  }
  f32x4 acc = zero;
#pragma unroll
  for (int u = 0; u < kSplitUnroll; ++u) acc += vx[u] + vb[u];
  float s = wave_sum((acc.x + acc.y) + (acc.z + acc.w));
  if ((t & (kWave - 1)) == 0) part[t >> 6] = s;
  __syncthreads();
  if (t == 0) partial[blockIdx.x] = (part[0] + part[1]) + (part[2] + part[3]);
}

// y[row] = the row's partial sums, lane l adding those at l, l + 64, ..., then the wave reduction
__global__ __launch_bounds__(kSplitThreads) void bcast_add_rowsum_f32_join(
    const float *__restrict__ partial, float *__restrict__ y, int64_t m, int parts) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t row = (int64_t)blockIdx.x * (kSplitThreads / kWave) + (threadIdx.x >> 6);
  if (row >= m) return;
  float s = 0.f;
  for (int p = lane; p < parts; p += kWave) s += partial[row * parts + p];
  s = wave_sum(s);
  if (lane == 0) y[row] = s;
}

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
float *g_scratch[kMaxDevices];   // per device: where that GPU keeps afir_rowsum_scratch

// The current device's copy of the scratch array (looked up on the first call per device).
LaunchStatus scratch_of_current_device(float **out) {
  int device = -1;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) return LaunchStatus{2u, hipGetErrorString(e)};
  if (device < 0 || device >= kMaxDevices) return invalid("broadcast_add_reducesum_noalloc: device ordinal out of range");
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch[device]) {
    float *p = nullptr;
    e = hipGetSymbolAddress(reinterpret_cast<void **>(&p), HIP_SYMBOL(afir_rowsum_scratch));
    if (e != hipSuccess || !p) {
      (void)hipGetLastError();
      return LaunchStatus{2u, e != hipSuccess ? hipGetErrorString(e) : "no address for the scratch array"};
    }
    g_scratch[device] = p;
  }
  *out = g_scratch[device];
  return ok_status();
}

}  // namespace
}  // namespace afir

extern "C" uint32_t afir_hip_launch_broadcast_add_reducesum_noalloc(uint32_t block_dim, void *stream, void *x,
                                                                    void *bias, void *y, void * /*workspace*/,
                                                                    void *tiling) {
  using namespace afir;
  // (errors: the code only; this entry point keeps no message and touches no heap)
  if (!tiling) return AFIR_HIP_E_INVALID;
  int64_t f[2];
  __builtin_memcpy(f, tiling, sizeof f);
  const int64_t m = f[0], n = f[1];
  if (m < 0 || n < 0) return AFIR_HIP_E_INVALID;
  if (m == 0) return AFIR_HIP_OK;
  if (!y || (n > 0 && (!x || !bias))) return AFIR_HIP_E_INVALID;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const bool vec = n > 0 && n % 4 == 0 && aligned16(x) && aligned16(bias);
  // few rows of at least two chunks: split and join through the scratch array
  if (vec && m < 1024 && n >= 2 * kSplitChunk && !block_dim) {
    const int64_t parts = (n + kSplitChunk - 1) / kSplitChunk;
    if (m * parts > kScratchFloats) return AFIR_HIP_E_NOALLOC_LIMIT;
    float *scratch = nullptr;
    const LaunchStatus got = scratch_of_current_device(&scratch);
    if (got.code) return got.code == 1 ? AFIR_HIP_E_INVALID : AFIR_HIP_E_LAUNCH;
    AFIR_LAUNCH("bcast_add_rowsum_f32_split", bcast_add_rowsum_f32_split, dim3((unsigned)(m * parts)), dim3(kSplitThreads), 0, st,
                       static_cast<const float *>(x), static_cast<const float *>(bias), scratch, n, (int)parts);
    AFIR_LAUNCH("bcast_add_rowsum_f32_join", bcast_add_rowsum_f32_join, dim3((unsigned)((m + 3) / 4)), dim3(kSplitThreads), 0, st,
                       scratch, static_cast<float *>(y), m, (int)parts);
    return hipGetLastError() == hipSuccess ? AFIR_HIP_OK : AFIR_HIP_E_LAUNCH;
  }
  // every other shape runs on kernels that need no scratch memory
  const LaunchStatus done = launch_broadcast_add_reducesum(static_cast<const float *>(x), static_cast<const float *>(bias),
                                                          static_cast<float *>(y), m, n, block_dim, st);
  return done.code == 0 ? AFIR_HIP_OK : done.code == 1 ? AFIR_HIP_E_INVALID : AFIR_HIP_E_LAUNCH;
}
