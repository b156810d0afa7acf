// Matmul with transposed and / or batched operands, same epilogue as matmul.hip:
//   out[b, m, n] = act(sum_k A(b, m, k) * B(b, k, n) + bias[n])
// where A lies in memory as [M, K] or, transposed, as [K, M], and B as [K, N] or
// [N, K]: linalg.matmul_transpose_a / _b and linalg.batch_matmul*, the other
// matmul-like ops the reference's recogniser takes
// (lib/Conversion/MarkStructuredOps/AnnotateMixMatmulSemanticsPass.cpp:244-256)
// and whose flags travel in its ABI as abi_matmul_trans_a / _b and the batch
// extent (lib/Runtime/Mix/MixAbi.cpp:293, lib/Runtime/Mix/MixTilingGenerator.cpp:
// 100-118).  The plain layout keeps its own kernels (matmul_dma.hip, matmul.hip).
//
// One workgroup (4 waves as 2 x 2) owns a 128 x 128 tile of one batch's output
// and walks K in steps of 64, two LDS stages, one barrier per step, as in
// matmul.hip.  Both operands sit in LDS with K innermost (rows of 128 data bytes
// + 16 pad bytes), whatever their layout in memory:
//   * an operand whose memory rows run along K (A as [M, K]; B as [N, K]) is copied
//     as it lies, one 16-byte chunk of eight K values per lane and load;
//   * an operand whose memory rows run along the other extent (B as [K, N]; A as
//     [K, M]) is transposed on the way: a lane fetches a 4 (k) x 8 block with four
//     128-bit loads, permutes the halves in registers and writes eight 64-bit words.
// Accesses are bounds-checked by 16-byte chunk, so M, K and N are arbitrary as long
// as every memory row starts on a 16-byte boundary (the contiguous extent of each
// operand and of the output a multiple of 8 elements, bases 16-byte aligned);
// anything else takes the element kernel below.  v_mfma_f32_32x32x16 with the
// operands swapped, so that a lane holds four consecutive n of one m for the
// epilogue.
#include <mutex>
#include <type_traits>

#include "kernels.h"

namespace afir {

namespace {

constexpr int kLK = 64;                 // K per step
constexpr int kLPitch = kLK * 2 + 16;   // bytes per LDS row
constexpr int kLT = 128;                // tile edge
constexpr int kLThreads = 256;

__device__ __forceinline__ uint32_t lperm_lo(uint32_t hi_row, uint32_t lo_row) {
  return __builtin_amdgcn_perm(hi_row, lo_row, 0x05040100u);
}
__device__ __forceinline__ uint32_t lperm_hi(uint32_t hi_row, uint32_t lo_row) {
  return __builtin_amdgcn_perm(hi_row, lo_row, 0x07060302u);
}

// An operand tile of 128 (rows of the output extent) x 64 (k) on its way to LDS.
// KC: memory rows run along K (element (x, k) at base[x * ld + k]).
struct TileKC {
  u32x4 r[kLT * 8 / kLThreads];   // 4 chunks per lane
  __device__ __forceinline__ void fetch(const uint16_t *base, int64_t ld, int x0, int extent, int k0, int K, int t) {
#pragma unroll
    for (int i = 0; i < kLT * 8 / kLThreads; ++i) {
      const int id = t + kLThreads * i, row = id >> 3, c = id & 7;
      const u32x4 zero4 = {0u, 0u, 0u, 0u};
      r[i] = (x0 + row < extent && k0 + c * 8 < K)
                 ? *reinterpret_cast<const u32x4 *>(base + (int64_t)(x0 + row) * ld + k0 + c * 8)
                 : zero4;
    }
  }
  __device__ __forceinline__ void stash(unsigned char *lds, int t) const {
#pragma unroll
    for (int i = 0; i < kLT * 8 / kLThreads; ++i) {
      const int id = t + kLThreads * i, row = id >> 3, c = id & 7;
      *reinterpret_cast<u32x4 *>(lds + row * kLPitch + c * 16) = r[i];
    }
  }
};
// KM: memory rows run along the output extent (element (x, k) at base[k * ld + x]).
struct TileKM {
  u32x4 r[4];                      // one 4 (k) x 8 (x) block per lane
  __device__ __forceinline__ static void where(int t, int &kg, int &xc) {
    const int half = t & 1, kq = (t >> 1) & 3, xcl = (t >> 3) & 7, rest = t >> 6;
    kg = (((rest & 1) * 4 + kq) << 1) + half;   // 0 .. 15: group of 4 k
    xc = (rest >> 1) * 8 + xcl;                 // 0 .. 15: chunk of 8 x
  }
  __device__ __forceinline__ void fetch(const uint16_t *base, int64_t ld, int x0, int extent, int k0, int K, int t) {
    int kg, xc;
    where(t, kg, xc);
    const u32x4 zero4 = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int q = 0; q < 4; ++q)
      r[q] = (k0 + kg * 4 + q < K && x0 + xc * 8 < extent)
                 ? *reinterpret_cast<const u32x4 *>(base + (int64_t)(k0 + kg * 4 + q) * ld + x0 + xc * 8)
                 : zero4;
  }
  __device__ __forceinline__ void stash(unsigned char *lds, int t) const {
    int kg, xc;
    where(t, kg, xc);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int d = j >> 1;
      u32x2 w;
      if (j & 1) {
        w.x = lperm_hi(r[1][d], r[0][d]);
        w.y = lperm_hi(r[3][d], r[2][d]);
      } else {
        w.x = lperm_lo(r[1][d], r[0][d]);
        w.y = lperm_lo(r[3][d], r[2][d]);
      }
      *reinterpret_cast<u32x2 *>(lds + (xc * 8 + j) * kLPitch + kg * 8) = w;
    }
  }
};

template <bool TA, bool TB, bool F16IO>
__global__ __launch_bounds__(kLThreads) void matmul_layout_mfma(
    const uint16_t *__restrict__ A, const uint16_t *__restrict__ B, const void *__restrict__ bias_v,
    void *__restrict__ out_v, int M, int K, int N, int64_t batch_a, int64_t batch_b, int64_t batch_out,
    float alpha, int relu, int tiles_m, int tiles_n) {
  constexpr int STAGE = 2 * kLT * kLPitch;   // A tile, then B tile
  extern __shared__ __align__(16) unsigned char smem[];
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int KT = (K + kLK - 1) / kLK;
  const uint16_t *a = A + (int64_t)blockIdx.y * batch_a;
  const uint16_t *b = B + (int64_t)blockIdx.y * batch_b;
  // A as [M, K]: rows along K, row pitch K.  A as [K, M]: rows along M, pitch M.
  const int64_t lda = TA ? M : K, ldb = TB ? K : N;
  typedef typename std::conditional<TA, TileKM, TileKC>::type TileA;
  typedef typename std::conditional<TB, TileKC, TileKM>::type TileB;

  for (int p = blockIdx.x; p < tiles_m * tiles_n; p += gridDim.x) {
    const int m0 = (p / tiles_n) * kLT, n0 = (p % tiles_n) * kLT;
    f32x16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

    TileA ta;
    TileB tb;
    auto compute = [&](int stage) {
      const unsigned char *As = smem + stage * STAGE;
      const unsigned char *Bs = As + kLT * kLPitch;
      const int lrow = lane & 31, lk = lane >> 5;
#pragma unroll
      for (int ks = 0; ks < kLK / 16; ++ks) {
        u32x4 fa[2], fb[2];
#pragma unroll
        for (int i = 0; i < 2; ++i)
          fa[i] = *reinterpret_cast<const u32x4 *>(As + ((wm * 2 + i) * 32 + lrow) * kLPitch + (ks * 2 + lk) * 16);
#pragma unroll
        for (int j = 0; j < 2; ++j)
          fb[j] = *reinterpret_cast<const u32x4 *>(Bs + ((wn * 2 + j) * 32 + lrow) * kLPitch + (ks * 2 + lk) * 16);
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
          for (int j = 0; j < 2; ++j) {
            if constexpr (F16IO)
              acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(
                  __builtin_bit_cast(f16x8, fb[j]), __builtin_bit_cast(f16x8, fa[i]), acc[i][j], 0, 0, 0);
            else
              acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                  __builtin_bit_cast(bf16x8, fb[j]), __builtin_bit_cast(bf16x8, fa[i]), acc[i][j], 0, 0, 0);
          }
      }
    };

    ta.fetch(a, lda, m0, M, 0, K, t);
    tb.fetch(b, ldb, n0, N, 0, K, t);
    ta.stash(smem, t);
    tb.stash(smem + kLT * kLPitch, t);
    __syncthreads();
    for (int kt = 0; kt < KT; ++kt) {
      const int cur = kt & 1;
      if (kt + 1 < KT) {
        ta.fetch(a, lda, m0, M, (kt + 1) * kLK, K, t);
        tb.fetch(b, ldb, n0, N, (kt + 1) * kLK, K, t);
      }
      compute(cur);
      if (kt + 1 < KT) {
        ta.stash(smem + (cur ^ 1) * STAGE, t);
        tb.stash(smem + (cur ^ 1) * STAGE + kLT * kLPitch, t);
      }
      __syncthreads();
    }

    // epilogue: lane holds m = lane % 32, n = 8 q + 4 (lane / 32) + e
    const int lm = lane & 31, lq = lane >> 5;
    unsigned char *const out_b = static_cast<unsigned char *>(out_v) + (int64_t)blockIdx.y * batch_out * (F16IO ? 4 : 2);
#pragma unroll
    for (int j = 0; j < 2; ++j) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int n = n0 + (wn * 2 + j) * 32 + 8 * q + 4 * lq;
        if (n >= N) continue;   // N is a multiple of 8 here: the four n of a lane are in or out together
        float b0, b1, b2, b3;
        if (!bias_v) {
          b0 = b1 = b2 = b3 = -0.f;   // no bias: x + (-0) is x for every x, signed zeros included
        } else if constexpr (F16IO) {
          const f32x4 bf = *reinterpret_cast<const f32x4 *>(static_cast<const float *>(bias_v) + n);
          b0 = bf[0]; b1 = bf[1]; b2 = bf[2]; b3 = bf[3];
        } else {
          const u32x2 braw = *reinterpret_cast<const u32x2 *>(static_cast<const uint16_t *>(bias_v) + n);
          b0 = bf16_lo(braw.x); b1 = bf16_hi(braw.x);
          b2 = bf16_lo(braw.y); b3 = bf16_hi(braw.y);
        }
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          const int m = m0 + (wm * 2 + i) * 32 + lm;
          if (m >= M) continue;
          float v0 = acc[i][j][4 * q + 0] + b0;
          float v1 = acc[i][j][4 * q + 1] + b1;
          float v2 = acc[i][j][4 * q + 2] + b2;
          float v3 = acc[i][j][4 * q + 3] + b3;
          v0 = fmaxf(v0, relu ? 0.f : v0 * alpha);
          v1 = fmaxf(v1, relu ? 0.f : v1 * alpha);
          v2 = fmaxf(v2, relu ? 0.f : v2 * alpha);
          v3 = fmaxf(v3, relu ? 0.f : v3 * alpha);
          if constexpr (F16IO) {
            const f32x4 w = {v0, v1, v2, v3};
            *reinterpret_cast<f32x4 *>(reinterpret_cast<float *>(out_b) + (int64_t)m * N + n) = w;
          } else {
            u32x2 w;
            w.x = pack_bf16(v0, v1);
            w.y = pack_bf16(v2, v3);
            *reinterpret_cast<u32x2 *>(reinterpret_cast<uint16_t *>(out_b) + (int64_t)m * N + n) = w;
          }
        }
      }
    }
    __syncthreads();   // the next tile's first stash must not overtake this tile's last reads
  }
}

// Any extents, any alignment: a 16 x 16 output tile per workgroup, f32 FMAs in the order of k.
template <bool F16IO>
__global__ __launch_bounds__(256) void matmul_layout_any(
    const uint16_t *__restrict__ A, const uint16_t *__restrict__ B, const void *__restrict__ bias_v,
    void *__restrict__ out_v, int M, int K, int N, int ta, int tb, int64_t batch_a, int64_t batch_b,
    int64_t batch_out, float alpha, int relu, int tiles_m, int tiles_n) {
  auto widen = [](uint16_t h) {
    if constexpr (F16IO) return (float)__builtin_bit_cast(_Float16, h);
    else return __uint_as_float((uint32_t)h << 16);
  };
  __shared__ float As[16][17], Bs[16][17];
  const uint16_t *a = A + (int64_t)blockIdx.y * batch_a;
  const uint16_t *b = B + (int64_t)blockIdx.y * batch_b;
  const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
  for (int p = blockIdx.x; p < tiles_m * tiles_n; p += gridDim.x) {
    const int m = (p / tiles_n) * 16 + ty, n = (p % tiles_n) * 16 + tx;
    float acc = 0.f;
    for (int k0 = 0; k0 < K; k0 += 16) {
      const int ka = k0 + tx, kb = k0 + ty;
      As[ty][tx] = (m < M && ka < K) ? widen(ta ? a[(int64_t)ka * M + m] : a[(int64_t)m * K + ka]) : 0.f;
      Bs[ty][tx] = (kb < K && n < N) ? widen(tb ? b[(int64_t)n * K + kb] : b[(int64_t)kb * N + n]) : 0.f;
      __syncthreads();
#pragma unroll
      for (int kk = 0; kk < 16; ++kk) acc += As[ty][kk] * Bs[kk][tx];
      __syncthreads();
    }
    if (m < M && n < N) {
      const int64_t o = (int64_t)blockIdx.y * batch_out + (int64_t)m * N + n;
      if constexpr (F16IO) {
        float v = acc + (bias_v ? static_cast<const float *>(bias_v)[n] : -0.f);
        static_cast<float *>(out_v)[o] = fmaxf(v, relu ? 0.f : v * alpha);
      } else {
        float v = acc + (bias_v ? __uint_as_float((uint32_t) static_cast<const uint16_t *>(bias_v)[n] << 16) : -0.f);
        v = fmaxf(v, relu ? 0.f : v * alpha);
        static_cast<uint16_t *>(out_v)[o] = (uint16_t)f32_to_bf16_rne(v);
      }
    }
  }
}

template <bool TA, bool TB, bool F16IO>
LaunchStatus launch_layout_mfma(const uint16_t *a, const uint16_t *b, const void *bias, void *out, int batch, int m,
                                int k, int n, float alpha, bool relu, uint32_t block_dim, hipStream_t stream) {
  constexpr size_t kLds = 2 * (size_t)2 * kLT * kLPitch;
  auto kernel = matmul_layout_mfma<TA, TB, F16IO>;
  static hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLds);
  if (attr != hipSuccess) return LaunchStatus{2u, hipGetErrorString(attr)};
  const int tiles_m = (m + kLT - 1) / kLT, tiles_n = (n + kLT - 1) / kLT;
  int64_t blocks = (int64_t)tiles_m * tiles_n;
  if (block_dim) blocks = block_dim;
  AFIR_LAUNCH("matmul_layout_mfma", kernel, dim3((unsigned)blocks, (unsigned)batch), dim3(kLThreads), kLds, stream, a, b, bias, out,
                     m, k, n, (int64_t)m * k, (int64_t)k * n, (int64_t)m * n, alpha, relu ? 1 : 0, tiles_m, tiles_n);
  return after_launch();
}

// ---- large products with a transposed operand: transpose it, then the direct-to-LDS kernel ----
//
// The direct-to-LDS kernel (matmul_dma_kernel.h) wants A as rows along K and B as rows along N.
// An operand stored the other way round is first brought into that form by an HBM-bound tiled
// transpose into scratch memory of the stream (a read and a write of the operand: 52 us for
// 8192 x 8192 16-bit elements against 750-770 us of multiplication), which then runs as it does
// for the plain layout: 6-7 % behind it, against 40-60 % behind on the register-staged kernel above.
// 64 x 64 tiles of 16-bit elements through LDS, 128-bit loads and stores on both sides.  In LDS an
// element takes a 32-bit word and a tile row 65 words: the eight words a lane writes per chunk and
// the eight it reads per output chunk then fall into different banks for every lane of a wave
// (neither this nor 16-bit writes into rows of 72 halves is what bounds the kernel: both measured
// the same; the order of the tiles below and the non-temporal loads are what moved it).
constexpr int kTrTile = 64, kTrPitch = 65;   // pitch in 32-bit words
constexpr int kTrBand = 32;
__global__ __launch_bounds__(256) void transpose_u16_tile64(const uint16_t *__restrict__ src, uint16_t *__restrict__ dst,
                                                            int rows, int cols) {
  __shared__ uint32_t tile[kTrTile * kTrPitch];   // [column of src][row of src]
  // Tiles in bands of kTrBand tile rows, a band walked down its rows first: the workgroups that
  // run together then cover runs of 4 KiB along the rows of dst and of 8 KiB along those of src.
  // Walked along the rows of src alone (runs of 16 KiB read, 128 bytes written at a pitch that
  // is a large power of two) the same kernel took 70 us for 8192 x 8192 instead of 52; bands of
  // 8 / 16 / 24 / 48 / 64 / all rows: 57 / 56 / 53.4 / 56 / 58 / 59.
  const int tiles_c = cols / kTrTile, tiles_r = rows / kTrTile;
  const int per_band = kTrBand * tiles_c;
  const int band = blockIdx.x / per_band, within = blockIdx.x - band * per_band;
  const int height = tiles_r - band * kTrBand < kTrBand ? tiles_r - band * kTrBand : kTrBand;
  const int tc = within / height, tr = band * kTrBand + (within - tc * height);
  src += (int64_t)blockIdx.y * rows * cols;   // one matrix per blockIdx.y, densely packed
  dst += (int64_t)blockIdx.y * rows * cols;
  const int t = threadIdx.x, chunk = t & 7, line = t >> 3;    // a lane moves two 16-byte chunks
  u32x4 v[2];
#pragma unroll
  for (int h = 0; h < 2; ++h)
    v[h] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(src + (int64_t)(tr * kTrTile + line + 32 * h) * cols + tc * kTrTile + chunk * 8));
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int r = line + 32 * h;
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      tile[(chunk * 8 + 2 * d) * kTrPitch + r] = v[h][d] & 0xffffu;
      tile[(chunk * 8 + 2 * d + 1) * kTrPitch + r] = v[h][d] >> 16;
    }
  }
  __syncthreads();
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int c = line + 32 * h;
    const uint32_t *w = tile + c * kTrPitch + chunk * 8;
    u32x4 o;
#pragma unroll
    for (int d = 0; d < 4; ++d) o[d] = w[2 * d] | (w[2 * d + 1] << 16);
    __builtin_nontemporal_store(o, reinterpret_cast<u32x4 *>(dst + (int64_t)(tc * kTrTile + c) * rows + tr * kTrTile + chunk * 8));
  }
}

// dst[z][c][r] = src[z][r][c] for `batch` rows x cols matrices of 16-bit elements (both multiples of 64)
void launch_transpose_u16(const uint16_t *src, uint16_t *dst, int64_t batch, int64_t rows, int64_t cols, hipStream_t stream) {
  const int64_t tiles = (rows / kTrTile) * (cols / kTrTile);
  AFIR_LAUNCH("transpose_u16_tile64", transpose_u16_tile64, dim3((unsigned)tiles, (unsigned)batch), dim3(256), 0, stream, src, dst,
              (int)rows, (int)cols);
}

// Scratch memory of the stream's order (hipMallocAsync): the device's default pool, told once
// to keep what is freed instead of returning it to the system at the next synchronisation.
void *stream_scratch(size_t bytes, hipStream_t stream) {
  static std::once_flag keep[64];
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= 64) {
    (void)hipGetLastError();
    return nullptr;
  }
  std::call_once(keep[device], [device] {
    hipMemPool_t pool = nullptr;
    uint64_t threshold = UINT64_MAX;
    if (hipDeviceGetDefaultMemPool(&pool, device) != hipSuccess ||
        hipMemPoolSetAttribute(pool, hipMemPoolAttrReleaseThreshold, &threshold) != hipSuccess)
      (void)hipGetLastError();
  });
  void *p = nullptr;
  if (hipMallocAsync(&p, bytes, stream) != hipSuccess) {
    (void)hipGetLastError();
    return nullptr;
  }
  return p;
}

// The direct-to-LDS kernel for transposed and / or batched operands, when the shape is one it
// takes and, with a transposed operand, the stream can allocate; false: not taken, nothing was
// launched.  A batch is a stack of products to that kernel (its tiles are dealt out over the whole
// stack), so sixteen products of 1024^3 fill the chip like one of 4096 x 1024 x 4096.
template <bool F16IO>
bool launch_on_dma(const uint16_t *a, const uint16_t *b, const void *bias, void *out, int64_t batch, int64_t m, int64_t k,
                   int64_t n, bool ta, bool tb, float alpha, bool relu, hipStream_t stream, LaunchStatus *status) {
  // (the same choice as the plain layout makes: products of fewer 256 x 256 tiles than half the
  // compute units keep to smaller tiles)
  if (!matmul_dma_supported(m, k, n) || batch * (m / 256) * (n / 256) < (int64_t)device_cus() / 2) return false;
  if (!env_int("AFIR_HIP_MATMUL_LAYOUTS_DIRECT", 1, 0, 1)) return false;   // 0: the register-staged kernel (to compare)
  // Two transposes cost 2 x 2 bytes x (m k + k n) of HBM traffic against 2 m k n flops: with both
  // operands transposed and products under 2048 x 2048 outputs they cost as much as the product
  // itself (16 x 1024^3: 445 TFLOP/s this way, 503 on the register-staged kernel; 8 x 2048^3: 794
  // against 685; 32 x 1024 x 4096 x 1024: 683 against 616).  One transposed operand measured
  // level or ahead on every shape tried (64 x 512^3: 376-392 against 339-382).
  if (ta && tb && !((m >= 2048 && n >= 2048) || k >= 4096)) return false;
  if (batch * m > 0x7fffffff || batch * (m / 256) * (n / 256) > 0x7fffffff) return false;
  if (!aligned16(a) || !aligned16(b) || !aligned16(out) || (reinterpret_cast<uintptr_t>(bias) & (F16IO ? 15u : 7u))) return false;
  uint16_t *at = nullptr, *bt = nullptr;
  if (ta || tb) {
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &capturing) != hipSuccess || capturing != hipStreamCaptureStatusNone) {
      (void)hipGetLastError();
      return false;   // no allocations inside a graph capture: the register-staged kernel
    }
    if (ta && !(at = static_cast<uint16_t *>(stream_scratch((size_t)batch * m * k * 2, stream)))) return false;
    if (tb && !(bt = static_cast<uint16_t *>(stream_scratch((size_t)batch * k * n * 2, stream)))) {
      if (at) (void)hipFreeAsync(at, stream);
      return false;
    }
    if (ta) launch_transpose_u16(a, at, batch, k, m, stream);   // stored [K, M] -> [M, K]
    if (tb) launch_transpose_u16(b, bt, batch, n, k, stream);   // stored [N, K] -> [K, N]
  }
  const uint16_t *pa = ta ? at : a, *pb = tb ? bt : b;
  if (batch > 1)
    *status = launch_matmul_dma_batched(pa, pb, bias, out, F16IO, (int)batch, (int)m, (int)k, (int)n, alpha, relu, stream);
  else if constexpr (F16IO)
    *status = launch_matmul_dma_f16(pa, pb, static_cast<const float *>(bias), static_cast<float *>(out), (int)m, (int)k,
                                    (int)n, alpha, relu, 0, stream);
  else
    *status = launch_matmul_dma(pa, pb, static_cast<const uint16_t *>(bias), static_cast<uint16_t *>(out), (int)m, (int)k,
                                (int)n, alpha, relu, 0, stream);
  if (at) (void)hipFreeAsync(at, stream);
  if (bt) (void)hipFreeAsync(bt, stream);
  return true;
}

template <bool F16IO>
LaunchStatus launch_layouts_io(const uint16_t *a, const uint16_t *b, const void *bias, void *out, int64_t batch,
                               int64_t m, int64_t k, int64_t n, bool ta, bool tb, float alpha, bool relu,
                               uint32_t block_dim, hipStream_t stream) {
  if (batch < 0 || m < 0 || k < 0 || n < 0) return invalid("matmul: negative extent");
  if (batch == 0 || m == 0 || n == 0) return ok_status();
  if (!out) return invalid("matmul: null tensor pointer");   // a null bias means "no bias"
  if (k > 0 && (!a || !b)) return invalid("matmul: null input matrix");
  if (m > 0x7fffffff || n > 0x7fffffff || k > 0x7fffffff || batch > 65535)
    return invalid("matmul: extent exceeds 2^31-1 (batch: 65535)");
  if (m * n > INT64_MAX / 4 / batch || (k && (m * k > INT64_MAX / 4 / batch || k * n > INT64_MAX / 4 / batch)))
    return invalid("matmul: extent overflow");
  const bool al = aligned16(a) && aligned16(b) && aligned16(out) &&
                  ((reinterpret_cast<uintptr_t>(bias) & (F16IO ? 15u : 7u)) == 0);
  // every memory row of A, B and out on a 16-byte boundary, in every batch
  const int64_t a_run = ta ? m : k, b_run = tb ? k : n;
  const bool rows16 = a_run % 8 == 0 && b_run % 8 == 0 && n % 8 == 0 && k >= 1 &&
                      (batch == 1 || ((m * k) % 8 == 0 && (k * n) % 8 == 0 && (m * n) % 8 == 0));
  const int64_t tiles = ((m + kLT - 1) / kLT) * ((n + kLT - 1) / kLT);
  if (!block_dim && (batch > 1 || ta || tb)) {
    LaunchStatus status = ok_status();
    if (launch_on_dma<F16IO>(a, b, bias, out, batch, m, k, n, ta, tb, alpha, relu, stream, &status)) return status;
  }
  if (al && rows16 && m * n >= 64 * 64 && tiles <= 0x7fffffff) {
    const int bi = (int)batch, mi = (int)m, ki = (int)k, ni = (int)n;
    if (ta && tb) return launch_layout_mfma<true, true, F16IO>(a, b, bias, out, bi, mi, ki, ni, alpha, relu, block_dim, stream);
    if (ta) return launch_layout_mfma<true, false, F16IO>(a, b, bias, out, bi, mi, ki, ni, alpha, relu, block_dim, stream);
    if (tb) return launch_layout_mfma<false, true, F16IO>(a, b, bias, out, bi, mi, ki, ni, alpha, relu, block_dim, stream);
    return launch_layout_mfma<false, false, F16IO>(a, b, bias, out, bi, mi, ki, ni, alpha, relu, block_dim, stream);
  }
  const int tiles_m = (int)((m + 15) / 16), tiles_n = (int)((n + 15) / 16);
  int64_t blocks = (int64_t)tiles_m * tiles_n;
  if (block_dim) blocks = block_dim;
  if (blocks > 0x7fffffff) blocks = 0x7fffffff;
  AFIR_LAUNCH("matmul_layout_any<F16IO>", matmul_layout_any<F16IO>, dim3((unsigned)blocks, (unsigned)batch), dim3(256), 0, stream, a, b,
                     bias, out, (int)m, (int)k, (int)n, ta ? 1 : 0, tb ? 1 : 0, m * k, k * n, m * n, alpha,
                     relu ? 1 : 0, tiles_m, tiles_n);
  return after_launch();
}

}  // namespace

LaunchStatus launch_matmul_layouts(const uint16_t *a, const uint16_t *b, const void *bias, void *out, bool f16io,
                                   int64_t batch, int64_t m, int64_t k, int64_t n, bool trans_a, bool trans_b,
                                   float alpha, bool relu, uint32_t block_dim, hipStream_t stream) {
  // the plain layout of one matrix pair has faster kernels of its own
  if (batch == 1 && !trans_a && !trans_b)
    return f16io ? launch_matmul_add_leakyrelu_f16(a, b, static_cast<const float *>(bias), static_cast<float *>(out), m,
                                                   k, n, alpha, relu, block_dim, stream)
                 : launch_matmul_add_leakyrelu(a, b, static_cast<const uint16_t *>(bias),
                                               static_cast<uint16_t *>(out), m, k, n, alpha, relu, block_dim, stream);
  return f16io ? launch_layouts_io<true>(a, b, bias, out, batch, m, k, n, trans_a, trans_b, alpha, relu, block_dim, stream)
               : launch_layouts_io<false>(a, b, bias, out, batch, m, k, n, trans_a, trans_b, alpha, relu, block_dim, stream);
}

}  // namespace afir
