// relu + broadcast add + transpose of the last two dims, f16:
//   out[b,j,i] = f16(relu(x[b,i,j]) + c[j]),  x [B,M,N] -> out [B,N,M]
// (parallel generic with a PureTranspose input map plus a PureBroadcast
// operand, lib/Conversion/LinalgToAscendC/ComputeConversion.cpp:265-333,
// 1290-1640; golden style examples/relu-broadcast-transpose/gen_inputs.py:34-35:
// f32 arithmetic, one round-to-nearest-even to f16).
//
// HBM-bound: 2 bytes in + 2 bytes out per element; the kernel for aligned
// shapes is described at its definition below.
#include "kernels.h"

namespace afir {

namespace {

constexpr int kThreads = 256;

// max(v, +0) with IEEE-754 maximum semantics: NaN propagates, -0 gives +0.
__device__ __forceinline__ float relu_keep_nan(float v) { return (v > 0.f) ? v : ((v != v) ? v : 0.f); }

// 64x64 tiles through a float32 LDS tile; a workgroup that walks several tiles has two in flight.
// Phase 1: a lane loads two 16-byte chunks of x rows (a wave covers eight
// 128-byte runs per load), applies relu and + c (its eight columns are fixed
// within a tile, so c is read once per tile) and writes the float32 results to
// tile[i][j], rows padded to 65 words.  Phase 2: a lane reads eight consecutive
// i of one j (a column of the padded tile: at most two lanes per bank), rounds
// them to f16 and writes one 16-byte chunk of an output row; eight lanes cover
// a 128-byte run along M.  The next tile's loads are issued before the current
// tile's stores, into the other of two LDS tiles, so a workgroup needs one
// barrier per tile and always has loads or stores outstanding.  Tiles are
// numbered along M first, so neighbouring workgroups write neighbouring runs
// of the same output rows.
//
// The loads are ordinary loads, the stores non-temporal (AFIR_TRANSPOSE_NT_LOADS, searched):
// with inputs that come from HBM the hint on the loads makes no difference here (23.7 against
// 23.9 us), and when a caller's inputs were read recently enough to sit in the 256 MB
// last-level cache, ordinary loads find them there (5.5 against 6.5 TB/s when the launches
// cycle over 256 MiB of inputs).
#ifndef AFIR_TRANSPOSE_NT_LOADS
#define AFIR_TRANSPOSE_NT_LOADS 0
#endif
#ifndef AFIR_TRANSPOSE_TILES_PER_WG
#define AFIR_TRANSPOSE_TILES_PER_WG 1
#endif
constexpr int kSmallTile = 64, kSmallPitch = kSmallTile + 1;
__global__ __launch_bounds__(kThreads) void relu_bcast_add_transpose_f16_tile64(
    const uint16_t *__restrict__ x, const uint16_t *__restrict__ c, uint16_t *__restrict__ out,
    int nb, int m, int n) {
  __shared__ float tiles[2][kSmallTile * kSmallPitch];
  const int t = threadIdx.x;
  // 32-bit tile numbers (the launcher checks that they fit): a 64-bit
  // division costs hundreds of instructions before the first load
  const unsigned tiles_m = (unsigned)(m / kSmallTile), tiles_n = (unsigned)(n / kSmallTile);
  const unsigned ntiles = (unsigned)nb * tiles_m * tiles_n;
  const int lj = (t & 7) * 8, li = t >> 3;        // phase 1: first column, row within a pass of 32
  const int oi = (t & 7) * 8, oj = t >> 3;        // phase 2: first i of the chunk, j within a pass of 32
  auto locate = [&](unsigned tile_id, int &m0, int &n0, int &b) {
    const unsigned rest = tile_id / tiles_m;
    m0 = (int)(tile_id - rest * tiles_m) * kSmallTile;
    b = (int)(rest / tiles_n);
    n0 = (int)(rest - (unsigned)b * tiles_n) * kSmallTile;
  };
  unsigned tile_id = blockIdx.x;
  if (tile_id >= ntiles) return;
  int m0, n0, b;
  locate(tile_id, m0, n0, b);
  u32x4 craw = *reinterpret_cast<const u32x4 *>(c + n0 + lj);
  u32x4 v[2];
  {
    const uint16_t *xin = x + ((int64_t)b * m + m0 + li) * n + n0 + lj;
#pragma unroll
    for (int k = 0; k < 2; ++k) v[k] = AFIR_TRANSPOSE_NT_LOADS ? load_nt(reinterpret_cast<const u32x4 *>(xin + (int64_t)(32 * k) * n))
                                      : *reinterpret_cast<const u32x4 *>(xin + (int64_t)(32 * k) * n);
  }
  int parity = 0;
  for (;;) {
    float *const tile = tiles[parity];
#pragma unroll
    for (int k = 0; k < 2; ++k)
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        float *dst = tile + (li + 32 * k) * kSmallPitch + lj + 2 * d;
        dst[0] = relu_keep_nan(f16_lo(v[k][d])) + f16_lo(craw[d]);
        dst[1] = relu_keep_nan(f16_hi(v[k][d])) + f16_hi(craw[d]);
      }
    // request the next tile before this one is written out
    const unsigned next_id = tile_id + gridDim.x;
    const bool more = next_id < ntiles;
    int next_m0 = 0, next_n0 = 0, next_b = 0;
    if (more) {
      locate(next_id, next_m0, next_n0, next_b);
      craw = *reinterpret_cast<const u32x4 *>(c + next_n0 + lj);
      const uint16_t *xin = x + ((int64_t)next_b * m + next_m0 + li) * n + next_n0 + lj;
#pragma unroll
      for (int k = 0; k < 2; ++k) v[k] = AFIR_TRANSPOSE_NT_LOADS ? load_nt(reinterpret_cast<const u32x4 *>(xin + (int64_t)(32 * k) * n))
                                      : *reinterpret_cast<const u32x4 *>(xin + (int64_t)(32 * k) * n);
    }
    // one barrier per tile: the other LDS tile was last read two barriers ago
    __syncthreads();
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      const int j = oj + 32 * k;
      u32x4 w;
#pragma unroll
      for (int d = 0; d < 4; ++d)
        w[d] = pack_f16(tile[(oi + 2 * d) * kSmallPitch + j], tile[(oi + 2 * d + 1) * kSmallPitch + j]);
      store_nt(reinterpret_cast<u32x4 *>(out + ((int64_t)b * n + n0 + j) * m + m0 + oi), w);
    }
    if (!more) break;
    tile_id = next_id;
    m0 = next_m0;
    n0 = next_n0;
    b = next_b;
    parity ^= 1;
  }
}

// The same tiles for shapes that fit the chip in one go (every lane of every workgroup resident
// at once: eight workgroups per CU, 64 registers, one LDS tile each), with the reads and the
// writes of the whole chip separated in time: HBM serves a pure read stream and a pure write
// stream faster than their mixture.  A workgroup takes four tiles that follow each other along N
// (it reads 512-byte runs; consecutive workgroups continue along N, so the requests of a moment
// fall into the same memory pages), requests all of them at once, transposes each as it arrives
// -- the LDS work sits in the shadow of the chip's reads -- and keeps the finished chunks in
// registers until `hold_ticks` of the real-time counter have passed since it started: by then
// the reads of all workgroups, which start within a microsecond or two of each other, have been
// served, and the stores leave back to back.  The wait is bounded and only shapes the timing:
// the stores are the same whenever they leave.  c is added after the transposition (a lane
// then needs one value per output row instead of eight per tile).
// Measured (us per launch, other kernel -> this one): [64, 1024, 512] 23.6 -> 21.3,
// [32, 1024, 512] 13.4 -> 11.0, [16, 2048, 1024] 23.9 -> 20.8, [4, 4096, 2048] 25.2 -> 21.9; the
// best hold is the time the bytes read take at AFIR_TRANSPOSE_PHASE_GBS plus
// AFIR_TRANSPOSE_PHASE_BASE_NS (5 % either side costs 2 %).  Below 24 MiB the other kernel is as
// fast or faster (one tile per workgroup spreads a small shape over more CUs) and stays in use;
// four tiles along M or 2 x 2 per workgroup measured 0.71 and 0.74 of peak at their best holds
// against 0.79.
#ifndef AFIR_TRANSPOSE_PHASED
#define AFIR_TRANSPOSE_PHASED 1
#endif
// a workgroup whose own loads came back so early that its place in the launch predicts the end of
// the chip's reads before this percentage of the formula's hold waits only until then
// (phase_hold_here; 100: the shorter of the two, 0: always the formula)
#ifndef AFIR_PHASE_ESTIMATE
#define AFIR_PHASE_ESTIMATE 100
#endif
#ifndef AFIR_TRANSPOSE_PHASE_GBS
#define AFIR_TRANSPOSE_PHASE_GBS 6900
#endif
#ifndef AFIR_TRANSPOSE_PHASE_BASE_NS
#define AFIR_TRANSPOSE_PHASE_BASE_NS 300
#endif
constexpr int kPhasedTiles = 4;           // tiles per workgroup, along N
constexpr int kPhasedLanesPerCU = 2048;
constexpr int kPhasedMinGroupsPerCU = 3;  // smaller launches take the other kernel
__global__ __launch_bounds__(kThreads, 8) void relu_bcast_add_transpose_f16_phased(
    const uint16_t *__restrict__ x, const uint16_t *__restrict__ c, uint16_t *__restrict__ out,
    int nb, int m, int n, int hold_ticks) {
  const long long t_start = wall_clock64();
  __shared__ float tile[kSmallTile * kSmallPitch];
  __shared__ float cs[kSmallTile * kPhasedTiles];
  const int t = threadIdx.x;
  const unsigned tiles_m = (unsigned)(m / kSmallTile), groups_n = (unsigned)(n / (kSmallTile * kPhasedTiles));
  const int lj = (t & 7) * 8, li = t >> 3;        // loads: first column, row within a pass of 32
  const int oi = (t & 7) * 8, oj = t >> 3;        // stores: first i of the chunk, j within a pass of 32
  const unsigned rest = blockIdx.x / groups_n;
  const int n0 = (int)(blockIdx.x - rest * groups_n) * (kSmallTile * kPhasedTiles);
  const int b = (int)(rest / tiles_m);
  const int m0 = (int)(rest - (unsigned)b * tiles_m) * kSmallTile;
  u32x4 v[kPhasedTiles][2];
  {
    const uint16_t *xin = x + ((int64_t)b * m + m0 + li) * n + n0 + lj;
#pragma unroll
    for (int q = 0; q < kPhasedTiles; ++q)
#pragma unroll
      for (int k = 0; k < 2; ++k)
        v[q][k] = *reinterpret_cast<const u32x4 *>(xin + (int64_t)(32 * k) * n + kSmallTile * q);
  }
  cs[t] = (float)__builtin_bit_cast(_Float16, c[n0 + t]);
#pragma unroll
  for (int q = 0; q < kPhasedTiles; ++q) {
#pragma unroll
    for (int k = 0; k < 2; ++k)
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        float *dst = tile + (li + 32 * k) * kSmallPitch + lj + 2 * d;
        dst[0] = relu_keep_nan(f16_lo(v[q][k][d]));
        dst[1] = relu_keep_nan(f16_hi(v[q][k][d]));
      }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      const int j = oj + 32 * k;
      const float cj = cs[kSmallTile * q + j];
#pragma unroll
      for (int d = 0; d < 4; ++d)
        v[q][k][d] = pack_f16(tile[(oi + 2 * d) * kSmallPitch + j] + cj, tile[(oi + 2 * d + 1) * kSmallPitch + j] + cj);
    }
    __syncthreads();
  }
  // (the asm makes the finished chunks exist here, so nothing of the above is left for after the hold)
#pragma unroll
  for (int q = 0; q < kPhasedTiles; ++q)
#pragma unroll
    for (int k = 0; k < 2; ++k) asm volatile("" : "+v"(v[q][k]));
#if AFIR_PHASE_ESTIMATE
  hold_ticks = phase_hold_here(hold_ticks, t_start, AFIR_PHASE_ESTIMATE * 0.01f);
#endif
  for (int spin = 0; spin < kPhaseSpinLimit && wall_clock64() - t_start < hold_ticks; ++spin)
    __builtin_amdgcn_s_sleep(1);
  // stores: a base per (tile, pass) that is the same for the whole workgroup (scalar registers)
  // plus one 32-bit offset per lane
  char *block_out = reinterpret_cast<char *>(out + ((int64_t)b * n + n0) * m + m0);
  const uint32_t lane_off = (uint32_t)(oj * m + oi) * 2u;
#pragma unroll
  for (int q = 0; q < kPhasedTiles; ++q)
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      char *base = block_out + (int64_t)(kSmallTile * q + 32 * k) * m * 2;
      // (s_nop: the store reads its four data registers over the following cycles)
      asm volatile("global_store_dwordx4 %0, %1, %2 nt\n\ts_nop 1" ::"v"(lane_off), "v"(v[q][k]), "s"(base) : "memory");
    }
}

// Any shape / alignment: 32x32 tiles through a padded LDS array, 2-byte accesses.
__global__ __launch_bounds__(kThreads) void relu_bcast_add_transpose_f16_any(
    const uint16_t *__restrict__ x, const uint16_t *__restrict__ c, uint16_t *__restrict__ out,
    int nb, int m, int n) {
  __shared__ uint16_t tile[32][33];
  const int tiles_m = (m + 31) / 32, tiles_n = (n + 31) / 32;
  const int64_t ntiles = (int64_t)nb * tiles_m * tiles_n;
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;  // 32 x 8
  for (int64_t tile_id = blockIdx.x; tile_id < ntiles; tile_id += gridDim.x) {
    const int tn = (int)(tile_id % tiles_n);
    const int tm = (int)((tile_id / tiles_n) % tiles_m);
    const int b = (int)(tile_id / ((int64_t)tiles_n * tiles_m));
    const int m0 = tm * 32, n0 = tn * 32;
    for (int r = ty; r < 32; r += 8) {
      int i = m0 + r, j = n0 + tx;
      if (i < m && j < n) {
        _Float16 xv = __builtin_bit_cast(_Float16, x[((int64_t)b * m + i) * n + j]);
        _Float16 cv = __builtin_bit_cast(_Float16, c[j]);
        _Float16 res = (_Float16)(relu_keep_nan((float)xv) + (float)cv);
        tile[r][tx] = __builtin_bit_cast(uint16_t, res);
      }
    }
    __syncthreads();
    for (int r = ty; r < 32; r += 8) {
      int j = n0 + r, i = m0 + tx;
      if (i < m && j < n) out[((int64_t)b * n + j) * m + i] = tile[tx][r];
    }
    __syncthreads();
  }
}

}  // namespace

LaunchStatus launch_relu_broadcast_add_transpose(const uint16_t *x, const uint16_t *c,
                                                 uint16_t *out, int64_t nb, int64_t m,
                                                 int64_t n, uint32_t block_dim,
                                                 hipStream_t stream) {
  if (nb < 0 || m < 0 || n < 0) return invalid("relu_broadcast_add_transpose: negative extent");
  if (nb == 0 || m == 0 || n == 0) return ok_status();
  if (!x || !c || !out) return invalid("relu_broadcast_add_transpose: null tensor pointer");
  if (nb > 0x7fffffff || m > 0x7fffffff || n > 0x7fffffff)
    return invalid("relu_broadcast_add_transpose: extent exceeds 2^31-1");
  if (nb > INT64_MAX / m / n / 4) return invalid("relu_broadcast_add_transpose: extent overflow");

  const bool tiled = (m % kSmallTile == 0) && (n % kSmallTile == 0) && aligned16(x) && aligned16(c) && aligned16(out) &&
                     nb * (m / kSmallTile) * (n / kSmallTile) < ((int64_t)1 << 31);
  // The phased kernel wants every lane of a launch resident at once: a shape of up to twice that
  // goes out as two launches of whole batches (kPhaseMaxLaunches).
  const int64_t groups_per_batch = tiled && n % (kSmallTile * kPhasedTiles) == 0 ? (m / kSmallTile) * (n / (kSmallTile * kPhasedTiles)) : 0;
  static const int fit = resident_blocks_per_cu(relu_bcast_add_transpose_f16_phased, kThreads, 0);   // workgroups per compute unit
  const int64_t capacity = fit >= kPhasedLanesPerCU / kThreads ? (int64_t)device_cus() * kPhasedLanesPerCU / kThreads : 0;   // groups per launch
  const int base_ns = env_int("AFIR_TRANSPOSE_PHASE_BASE_NS", AFIR_TRANSPOSE_PHASE_BASE_NS, 0, 100000);
  const int gbs = env_int("AFIR_TRANSPOSE_PHASE_GBS", AFIR_TRANSPOSE_PHASE_GBS, 100, 100000);
  if (AFIR_TRANSPOSE_PHASED && !block_dim && groups_per_batch > 0 && groups_per_batch <= capacity &&
      nb * groups_per_batch >= (int64_t)device_cus() * kPhasedMinGroupsPerCU && (int64_t)32 * m * 2 < ((int64_t)1 << 31) &&
      (nb + capacity / groups_per_batch - 1) / (capacity / groups_per_batch) <= kPhaseMaxLaunches && phased_enabled()) {
    const int64_t batches_per_launch = capacity / groups_per_batch;
    const int64_t launches = (nb + batches_per_launch - 1) / batches_per_launch;
    const int64_t take = (nb + launches - 1) / launches;
    for (int64_t b0 = 0; b0 < nb; b0 += take) {
      const int64_t nbl = nb - b0 < take ? nb - b0 : take;
      const int hold_ticks = phase_hold_ticks(nbl * m * n * 2, base_ns, gbs);
      AFIR_LAUNCH("relu_bcast_add_transpose_f16_phased", relu_bcast_add_transpose_f16_phased, dim3((unsigned)(nbl * groups_per_batch)), dim3(kThreads), 0,
                         stream, x + b0 * m * n, c, out + b0 * m * n, (int)nbl, (int)m, (int)n, hold_ticks);
    }
  } else if (tiled) {
    // one tile per workgroup: the hardware deals workgroups out as slots free up, which balances
    // better than walks of several tiles (8192 workgroups of one tile 19.7 us on [64, 1024, 512],
    // 4096 of two 20.4, 2731 of three 20.9; a grid given by the caller makes a workgroup walk,
    // with the next tile's loads in flight).  The two LDS tiles then also hold a CU to four
    // workgroups, which measured faster than the eight that one tile allows (20.7 us).
    int64_t blocks = (nb * (m / kSmallTile) * (n / kSmallTile) + AFIR_TRANSPOSE_TILES_PER_WG - 1) / AFIR_TRANSPOSE_TILES_PER_WG;
    if (blocks > (int64_t)device_cus() * 256) blocks = (int64_t)device_cus() * 256;
    if (block_dim) blocks = block_dim;
    AFIR_LAUNCH("relu_bcast_add_transpose_f16_tile64", relu_bcast_add_transpose_f16_tile64, dim3((unsigned)blocks), dim3(kThreads), 0, stream,
                       x, c, out, (int)nb, (int)m, (int)n);
  } else {
    int64_t blocks = nb * ((m + 31) / 32) * ((n + 31) / 32);
    if (block_dim) blocks = block_dim;
    if (blocks > 0x7fffffff) blocks = 0x7fffffff;
    AFIR_LAUNCH("relu_bcast_add_transpose_f16_any", relu_bcast_add_transpose_f16_any, dim3((unsigned)blocks), dim3(kThreads),
                       0, stream, x, c, out, (int)nb, (int)m, (int)n);
  }
  return after_launch();
}

}  // namespace afir
