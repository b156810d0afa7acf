// relu + broadcast add + transpose of the last two dims, f16:
//   out[b,j,i] = f16(relu(x[b,i,j]) + c[j]),  x [B,M,N] -> out [B,N,M]
// (parallel generic with a PureTranspose input map plus a PureBroadcast
// operand, lib/Conversion/LinalgToAscendC/ComputeConversion.cpp:265-333,
// 1290-1640; golden style examples/relu-broadcast-transpose/gen_inputs.py:34-35:
// f32 arithmetic, one round-to-nearest-even to f16).
//
// HBM-bound: 2 bytes in + 2 bytes out per element.  A workgroup of 256 lanes
// moves one 128x128 tile:
//   1. 128-bit global loads along N (16 lanes cover 256 contiguous bytes),
//      relu + c applied in registers (a lane's column chunk is the same for
//      all its rows, so its 8 values of c are loaded once), 128-bit LDS
//      writes;
//   2. every lane reads one 8x8 block back as eight 128-bit LDS reads,
//      transposes it in registers with byte permutes, and issues eight
//      128-bit global stores along M (16 lanes cover 256 contiguous bytes).
// The LDS tile is 128 rows x 256 B with no padding; the 16-byte chunk column
// is XOR-ed with (row/8)%16, which makes both the row-wise writes and the
// block-column reads hit 16 distinct bank groups per 16 lanes.
// The grid is persistent (a few workgroups per CU); each workgroup issues the
// loads of its next tile before it stores the current one, so HBM reads and
// writes overlap instead of alternating in phases.
#include "kernels.h"

namespace afir {

namespace {

#ifndef AFIR_TR_EXTRA_LDS
#define AFIR_TR_EXTRA_LDS 0
#endif
#ifndef AFIR_TR_BLOCKS_PER_CU
#define AFIR_TR_BLOCKS_PER_CU 5
#endif
constexpr int kThreads = 256;
constexpr int kTile = 128;               // elements per tile edge
constexpr int kChunksPerRow = kTile / 8;  // 16-byte chunks per LDS row

// max(v, +0) with IEEE-754 maximum semantics: NaN propagates, -0 gives +0.
__device__ __forceinline__ float relu_keep_nan(float v) { return (v > 0.f) ? v : ((v != v) ? v : 0.f); }

__device__ __forceinline__ uint32_t relu_add_pack(uint32_t packed, float c_lo, float c_hi) {
  float lo = relu_keep_nan(f16_lo(packed)) + c_lo;
  float hi = relu_keep_nan(f16_hi(packed)) + c_hi;
  return pack_f16(lo, hi);
}

__global__ __launch_bounds__(kThreads) void relu_bcast_add_transpose_f16_tiled(
    const uint16_t *__restrict__ x, const uint16_t *__restrict__ c, uint16_t *__restrict__ out,
    int nb, int m, int n) {
  __shared__ u32x4 tile[kTile * kChunksPerRow];  // 32 KiB

  const int tiles_m = m / kTile, tiles_n = n / kTile;
  const int64_t ntiles = (int64_t)nb * tiles_m * tiles_n;
  const int t = threadIdx.x;
  const int cc = t & 15;       // chunk column of this lane in the load phase
  const int row0 = t >> 4;     // first row of this lane in the load phase
  const int iblk = t & 15;     // 8-row block (along M) in the store phase
  const int jblk = t >> 4;     // 8-col block (along N) in the store phase

  // Software pipeline over the tiles of this workgroup: the global loads of
  // the next tile are issued before the current tile is read back from LDS and
  // stored, so reads and writes to HBM overlap instead of alternating.
  auto decode = [&](int64_t tile_id, int &b, int &m0, int &n0) {
    const int tn = (int)(tile_id % tiles_n);
    const int tm = (int)((tile_id / tiles_n) % tiles_m);
    b = (int)(tile_id / ((int64_t)tiles_n * tiles_m));
    m0 = tm * kTile;
    n0 = tn * kTile;
  };
  u32x4 v[8], craw;
  auto fetch = [&](int64_t tile_id) {
    int b, m0, n0;
    decode(tile_id, b, m0, n0);
    craw = *reinterpret_cast<const u32x4 *>(c + n0 + cc * 8);
    const uint16_t *xin = x + ((int64_t)b * m + m0) * n + n0 + cc * 8;
#pragma unroll
    for (int k = 0; k < 8; ++k)
      v[k] = load_nt(reinterpret_cast<const u32x4 *>(xin + (int64_t)(row0 + 16 * k) * n));
  };

  int64_t tile_id = blockIdx.x;
  if (tile_id < ntiles) fetch(tile_id);
  for (; tile_id < ntiles; tile_id += gridDim.x) {
    int b, m0, n0;
    decode(tile_id, b, m0, n0);
    float cf[8];
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      cf[2 * d] = f16_lo(craw[d]);
      cf[2 * d + 1] = f16_hi(craw[d]);
    }
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const int row = row0 + 16 * k;
      u32x4 r;
#pragma unroll
      for (int d = 0; d < 4; ++d) r[d] = relu_add_pack(v[k][d], cf[2 * d], cf[2 * d + 1]);
      tile[row * kChunksPerRow + (cc ^ ((row >> 3) & 15))] = r;
    }
    __syncthreads();
    if (tile_id + gridDim.x < ntiles) fetch(tile_id + gridDim.x);

    u32x4 in[8];
#pragma unroll
    for (int r = 0; r < 8; ++r) in[r] = tile[(iblk * 8 + r) * kChunksPerRow + (jblk ^ iblk)];

    uint16_t *o = out + ((int64_t)b * n + n0 + jblk * 8) * m + m0 + iblk * 8;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      u32x4 w;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        uint32_t xlo = in[2 * q][j >> 1], xhi = in[2 * q + 1][j >> 1];
        w[q] = (j & 1) ? __builtin_amdgcn_perm(xhi, xlo, 0x07060302u)
                       : __builtin_amdgcn_perm(xhi, xlo, 0x05040100u);
      }
      store_nt(reinterpret_cast<u32x4 *>(o + (int64_t)j * m), w);
    }
    __syncthreads();
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

  const bool tiled = (m % kTile == 0) && (n % kTile == 0) && aligned16(x) && aligned16(c) &&
                     aligned16(out);
  int64_t tiles = tiled ? nb * (m / kTile) * (n / kTile)
                        : nb * ((m + 31) / 32) * ((n + 31) / 32);
  int64_t blocks = tiles;
  if (AFIR_TR_BLOCKS_PER_CU && tiled && blocks > (int64_t)kNumCU * AFIR_TR_BLOCKS_PER_CU)
    blocks = (int64_t)kNumCU * AFIR_TR_BLOCKS_PER_CU;
  if (block_dim) blocks = block_dim;
  if (blocks > 0x7fffffff) blocks = 0x7fffffff;
  if (tiled) {
    hipLaunchKernelGGL(relu_bcast_add_transpose_f16_tiled, dim3((unsigned)blocks), dim3(kThreads),
                       AFIR_TR_EXTRA_LDS, stream, x, c, out, (int)nb, (int)m, (int)n);
  } else {
    hipLaunchKernelGGL(relu_bcast_add_transpose_f16_any, dim3((unsigned)blocks), dim3(kThreads),
                       0, stream, x, c, out, (int)nb, (int)m, (int)n);
  }
  return after_launch();
}

}  // namespace afir
