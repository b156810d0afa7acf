// Matmul + bias + leaky relu, bf16 in / f32 accumulate / bf16 out:
//   out = bf16(max(v, v*alpha)),  v = A[M,K] @ B[K,N] + bias[N]
// (mix kernel of lib/Target/CannKernel/CannTranslation.cpp:1573-1628,1848-1869;
// IR examples/matmul-add-leakyrelu/step0_input.mlir:22-52; golden
// examples/matmul-add-leakyrelu/gen_data.py:33-36 restated for bf16).
//
// MFMA-bound.  One workgroup owns a BM x BN tile of the output and walks K in
// steps of 64.  Per step the A tile [BM][64] is copied to LDS as it lies in
// memory; the B tile [64][BN] is transposed on the way (each lane fetches a
// 4(k) x 8(n) block with four 128-bit loads, permutes bytes in registers and
// writes eight 64-bit LDS words), so that both MFMA operands are eight
// K-contiguous bf16 values = one 128-bit LDS read per lane.  LDS rows are 128
// data bytes + 16 pad bytes, which spreads the 32 rows of an operand read
// over all banks.  Two LDS stages: the next K step is fetched into registers
// before the MFMAs of the current step are issued and written to the other
// stage afterwards, one barrier per step.
//
// The MFMA is v_mfma_f32_32x32x16_bf16 with the operands swapped (B^T tile
// as the row operand, A tile as the column operand), so a lane ends up holding
// four consecutive n for one m: the epilogue adds bias, applies max(v, v*alpha)
// in f32, rounds once to bf16 and stores 64 bits per lane.
//
// Workgroup ids are remapped so that the 32 workgroups resident on one XCD
// (ids congruent mod 8) form a compact patch of output tiles and share their A
// and B panels through that XCD's L2.
#include "kernels.h"

namespace afir {

namespace {

constexpr int kBK = 64;
constexpr int kPitch = kBK * 2 + 16;  // bytes per LDS row

__device__ __forceinline__ uint32_t perm_lo(uint32_t hi_row, uint32_t lo_row) {
  return __builtin_amdgcn_perm(hi_row, lo_row, 0x05040100u);
}
__device__ __forceinline__ uint32_t perm_hi(uint32_t hi_row, uint32_t lo_row) {
  return __builtin_amdgcn_perm(hi_row, lo_row, 0x07060302u);
}

__device__ __forceinline__ void map_tile(int p, int tiles_m, int tiles_n, int &tm, int &tn) {
  const int ntiles = tiles_m * tiles_n;
  int q = p;
  if ((ntiles % kNumXCD) == 0) q = (p % kNumXCD) * (ntiles / kNumXCD) + p / kNumXCD;
  constexpr int kGroupM = 4;
  const int per_group = kGroupM * tiles_n;
  const int group = q / per_group, within = q % per_group;
  const int first_m = group * kGroupM;
  const int gsize = (tiles_m - first_m < kGroupM) ? tiles_m - first_m : kGroupM;
  tm = first_m + within % gsize;
  tn = within / gsize;
}

// F16IO = false: A, B, bias, out are bf16.  F16IO = true: A, B are f16, bias
// and out are f32 -- the types of the reference's own matmul example
// (examples/matmul-add-leakyrelu/step0_input.mlir:10-15); same tiling, the
// f16 MFMA, and an epilogue that stores the float32 value unrounded.
// Eight consecutive 16-bit elements, the first `valid` of them read one by one
// (no alignment needed), the rest zeros.
__device__ __forceinline__ u32x4 load_elements(const uint16_t *p, int valid) {
  uint32_t h[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) h[e] = e < valid ? (uint32_t)p[e] : 0u;
  const u32x4 v = {h[0] | (h[1] << 16), h[2] | (h[3] << 16), h[4] | (h[5] << 16), h[6] | (h[7] << 16)};
  return v;
}

// EDGE = 1: M is arbitrary, K and N are multiples of 8 (rows start on 16-byte
// boundaries): chunks outside the matrices are read as zeros, stores outside
// are dropped, the K loop runs over the last, partly empty step as well.
// EDGE = 2: any M, K, N and any alignment: the same with element accesses.
template <int WAVES_M, int WAVES_N, int TM, int TN, bool F16IO, int EDGE>
__global__ __launch_bounds__(WAVES_M *WAVES_N * 64) void matmul_bias_leakyrelu_mfma(
    const uint16_t *__restrict__ A, const uint16_t *__restrict__ B,
    const void *__restrict__ bias_v, void *__restrict__ out_v, int M, int K, int N,
    float alpha, int relu, int tiles_m, int tiles_n) {
  constexpr int NT = WAVES_M * WAVES_N * 64;
  constexpr int BM = WAVES_M * TM * 32, BN = WAVES_N * TN * 32;
  constexpr int A_STAGE = BM * kPitch, B_STAGE = BN * kPitch, STAGE = A_STAGE + B_STAGE;
  constexpr int A_ITERS = BM * 8 / NT;              // 16-byte chunks of A per lane per step
  constexpr int B_ITERS = 16 * (BN / 8) / NT;       // 4x8 blocks of B per lane per step
  static_assert(A_ITERS >= 1 && B_ITERS >= 1, "tile too small for the workgroup");
  static_assert((BM * 8) % NT == 0 && (16 * (BN / 8)) % NT == 0, "uneven loader split");
  extern __shared__ __align__(16) unsigned char smem[];

  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;
  const int KT = EDGE ? (K + kBK - 1) / kBK : K / kBK;
  const u32x4 zero4 = {0u, 0u, 0u, 0u};

  for (int p = blockIdx.x; p < tiles_m * tiles_n; p += gridDim.x) {
    int tile_m, tile_n;
    map_tile(p, tiles_m, tiles_n, tile_m, tile_n);
    const int m0 = tile_m * BM, n0 = tile_n * BN;

    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

    u32x4 ra[A_ITERS];
    u32x4 rb[B_ITERS][4];

    auto fetch = [&](int kt) {
      const int k0 = kt * kBK;
#pragma unroll
      for (int i = 0; i < A_ITERS; ++i) {
        const int id = t + NT * i, row = id >> 3, c = id & 7;
        if (EDGE == 2) {
          const int left = m0 + row < M ? K - (k0 + c * 8) : 0;
          ra[i] = left > 0 ? load_elements(A + (int64_t)(m0 + row) * K + k0 + c * 8, left) : zero4;
        } else if (!EDGE || (m0 + row < M && k0 + c * 8 < K)) {
          ra[i] = *reinterpret_cast<const u32x4 *>(A + (int64_t)(m0 + row) * K + k0 + c * 8);
        } else {
          ra[i] = zero4;
        }
      }
#pragma unroll
      for (int i = 0; i < B_ITERS; ++i) {
        const int bi = t + NT * i;
        const int half = bi & 1, kq = (bi >> 1) & 3, ncl = (bi >> 3) & 7, rest = bi >> 6;
        const int kg = (((rest & 1) * 4 + kq) << 1) + half;
        const int nc = (rest >> 1) * 8 + ncl;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          if (EDGE == 2) {
            const int left = k0 + kg * 4 + r < K ? N - (n0 + nc * 8) : 0;
            rb[i][r] = left > 0 ? load_elements(B + (int64_t)(k0 + kg * 4 + r) * N + n0 + nc * 8, left) : zero4;
          } else if (!EDGE || (k0 + kg * 4 + r < K && n0 + nc * 8 < N)) {
            rb[i][r] = *reinterpret_cast<const u32x4 *>(B + (int64_t)(k0 + kg * 4 + r) * N + n0 + nc * 8);
          } else {
            rb[i][r] = zero4;
          }
        }
      }
    };

    auto stash = [&](int stage) {
      unsigned char *As = smem + stage * STAGE;
      unsigned char *Bs = As + A_STAGE;
#pragma unroll
      for (int i = 0; i < A_ITERS; ++i) {
        const int id = t + NT * i, row = id >> 3, c = id & 7;
        *reinterpret_cast<u32x4 *>(As + row * kPitch + c * 16) = ra[i];
      }
#pragma unroll
      for (int i = 0; i < B_ITERS; ++i) {
        const int bi = t + NT * i;
        const int half = bi & 1, kq = (bi >> 1) & 3, ncl = (bi >> 3) & 7, rest = bi >> 6;
        const int kg = (((rest & 1) * 4 + kq) << 1) + half;
        const int nc = (rest >> 1) * 8 + ncl;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int d = j >> 1;
          u32x2 w;
          if (j & 1) {
            w.x = perm_hi(rb[i][1][d], rb[i][0][d]);
            w.y = perm_hi(rb[i][3][d], rb[i][2][d]);
          } else {
            w.x = perm_lo(rb[i][1][d], rb[i][0][d]);
            w.y = perm_lo(rb[i][3][d], rb[i][2][d]);
          }
          *reinterpret_cast<u32x2 *>(Bs + (nc * 8 + j) * kPitch + kg * 8) = w;
        }
      }
    };

    auto compute = [&](int stage) {
      const unsigned char *As = smem + stage * STAGE;
      const unsigned char *Bs = As + A_STAGE;
      const int lrow = lane & 31, lk = lane >> 5;
#pragma unroll
      for (int ks = 0; ks < kBK / 16; ++ks) {
        u32x4 fa[TM], fb[TN];
#pragma unroll
        for (int i = 0; i < TM; ++i)
          fa[i] = *reinterpret_cast<const u32x4 *>(As + ((wm * TM + i) * 32 + lrow) * kPitch +
                                                   (ks * 2 + lk) * 16);
#pragma unroll
        for (int j = 0; j < TN; ++j)
          fb[j] = *reinterpret_cast<const u32x4 *>(Bs + ((wn * TN + j) * 32 + lrow) * kPitch +
                                                   (ks * 2 + lk) * 16);
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j) {
            if constexpr (F16IO)
              acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(
                  __builtin_bit_cast(f16x8, fb[j]), __builtin_bit_cast(f16x8, fa[i]), acc[i][j], 0, 0, 0);
            else
              acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                  __builtin_bit_cast(bf16x8, fb[j]), __builtin_bit_cast(bf16x8, fa[i]), acc[i][j], 0, 0, 0);
          }
      }
    };

    fetch(0);
    stash(0);
    __syncthreads();
    for (int kt = 0; kt < KT; ++kt) {
      const int cur = kt & 1;
      if (kt + 1 < KT) fetch(kt + 1);
      compute(cur);
      if (kt + 1 < KT) stash(cur ^ 1);
      __syncthreads();
    }

    // epilogue: lane holds m = lane%32, n = 8q + 4*(lane/32) + e
    const int lm = lane & 31, lq = lane >> 5;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int n = n0 + (wn * TN + j) * 32 + 8 * q + 4 * lq;
        float b0, b1, b2, b3;
        if (!bias_v || (EDGE && n >= N)) {
          b0 = b1 = b2 = b3 = -0.f;   // no bias: x + (-0) is x for every x, signed zeros included
        } else if (EDGE == 2) {
          float bb[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            if (n + e >= N) bb[e] = -0.f;
            else if constexpr (F16IO) bb[e] = static_cast<const float *>(bias_v)[n + e];
            else bb[e] = __uint_as_float((uint32_t) static_cast<const uint16_t *>(bias_v)[n + e] << 16);
          }
          b0 = bb[0]; b1 = bb[1]; b2 = bb[2]; b3 = bb[3];
        } else if constexpr (F16IO) {
          const f32x4 bf = *reinterpret_cast<const f32x4 *>(static_cast<const float *>(bias_v) + n);
          b0 = bf[0]; b1 = bf[1]; b2 = bf[2]; b3 = bf[3];
        } else {
          const u32x2 braw = *reinterpret_cast<const u32x2 *>(static_cast<const uint16_t *>(bias_v) + n);
          b0 = bf16_lo(braw.x); b1 = bf16_hi(braw.x);
          b2 = bf16_lo(braw.y); b3 = bf16_hi(braw.y);
        }
#pragma unroll
        for (int i = 0; i < TM; ++i) {
          const int m = m0 + (wm * TM + i) * 32 + lm;
          if (EDGE && (m >= M || n >= N)) continue;
          float v0 = acc[i][j][4 * q + 0] + b0;
          float v1 = acc[i][j][4 * q + 1] + b1;
          float v2 = acc[i][j][4 * q + 2] + b2;
          float v3 = acc[i][j][4 * q + 3] + b3;
          v0 = fmaxf(v0, relu ? 0.f : v0 * alpha);
          v1 = fmaxf(v1, relu ? 0.f : v1 * alpha);
          v2 = fmaxf(v2, relu ? 0.f : v2 * alpha);
          v3 = fmaxf(v3, relu ? 0.f : v3 * alpha);
          if (EDGE == 2) {
            const float vv[4] = {v0, v1, v2, v3};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              if (n + e >= N) continue;
              if constexpr (F16IO) static_cast<float *>(out_v)[(int64_t)m * N + n + e] = vv[e];
              else static_cast<uint16_t *>(out_v)[(int64_t)m * N + n + e] = (uint16_t)f32_to_bf16_rne(vv[e]);
            }
          } else if constexpr (F16IO) {
            const f32x4 w = {v0, v1, v2, v3};
            *reinterpret_cast<f32x4 *>(static_cast<float *>(out_v) + (int64_t)m * N + n) = w;
          } else {
            u32x2 w;
            w.x = pack_bf16(v0, v1);
            w.y = pack_bf16(v2, v3);
            *reinterpret_cast<u32x2 *>(static_cast<uint16_t *>(out_v) + (int64_t)m * N + n) = w;
          }
        }
      }
    }
  }
}

// Any shape: 16x16 output tile per workgroup, f32 FMAs, bounds-checked.
template <bool F16IO>
__global__ __launch_bounds__(256) void matmul_bias_leakyrelu_any(
    const uint16_t *__restrict__ A, const uint16_t *__restrict__ B,
    const void *__restrict__ bias_v, void *__restrict__ out_v, int M, int K, int N,
    float alpha, int relu, int tiles_m, int tiles_n) {
  auto widen = [](uint16_t h) {
    if constexpr (F16IO) return (float)__builtin_bit_cast(_Float16, h);
    else return __uint_as_float((uint32_t)h << 16);
  };
  __shared__ float As[16][17], Bs[16][17];
  const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
  for (int p = blockIdx.x; p < tiles_m * tiles_n; p += gridDim.x) {
    const int m = (p / tiles_n) * 16 + ty, n = (p % tiles_n) * 16 + tx;
    float acc = 0.f;
    for (int k0 = 0; k0 < K; k0 += 16) {
      const int ka = k0 + tx, kb = k0 + ty;
      As[ty][tx] = (m < M && ka < K) ? widen(A[(int64_t)m * K + ka]) : 0.f;
      Bs[ty][tx] = (kb < K && n < N) ? widen(B[(int64_t)kb * N + n]) : 0.f;
      __syncthreads();
#pragma unroll
      for (int kk = 0; kk < 16; ++kk) acc += As[ty][kk] * Bs[kk][tx];
      __syncthreads();
    }
    if (m < M && n < N) {
      if constexpr (F16IO) {
        float v = acc + (bias_v ? static_cast<const float *>(bias_v)[n] : -0.f);
        static_cast<float *>(out_v)[(int64_t)m * N + n] = fmaxf(v, relu ? 0.f : v * alpha);
      } else {
        float v = acc + (bias_v ? __uint_as_float((uint32_t) static_cast<const uint16_t *>(bias_v)[n] << 16) : -0.f);
        v = fmaxf(v, relu ? 0.f : v * alpha);
        static_cast<uint16_t *>(out_v)[(int64_t)m * N + n] = (uint16_t)f32_to_bf16_rne(v);
      }
    }
  }
}

template <int WAVES_M, int WAVES_N, int TM, int TN, bool F16IO, int EDGE = 0>
LaunchStatus launch_mfma(const uint16_t *a, const uint16_t *b, const void *bias, void *out, int m,
                         int k, int n, float alpha, bool relu, uint32_t block_dim, hipStream_t stream) {
  constexpr int NT = WAVES_M * WAVES_N * 64;
  constexpr int BM = WAVES_M * TM * 32, BN = WAVES_N * TN * 32;
  constexpr size_t kLds = 2 * (size_t)(BM + BN) * kPitch;
  auto kernel = matmul_bias_leakyrelu_mfma<WAVES_M, WAVES_N, TM, TN, F16IO, EDGE>;
  static hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                               hipFuncAttributeMaxDynamicSharedMemorySize,
                                               (int)kLds);
  if (attr != hipSuccess) return LaunchStatus{2u, hipGetErrorString(attr)};
  const int tiles_m = EDGE ? (m + BM - 1) / BM : m / BM, tiles_n = EDGE ? (n + BN - 1) / BN : n / BN;
  int64_t blocks = (int64_t)tiles_m * tiles_n;
  if (block_dim) blocks = block_dim;
  AFIR_LAUNCH("matmul_bias_leakyrelu_mfma", kernel, dim3((unsigned)blocks), dim3(NT), kLds, stream, a, b, bias, out, m, k,
                     n, alpha, relu ? 1 : 0, tiles_m, tiles_n);
  return after_launch();
}

}  // namespace

namespace {

template <bool F16IO>
LaunchStatus launch_matmul_any_io(const uint16_t *a, const uint16_t *b, const void *bias, void *out,
                                  int64_t m, int64_t k, int64_t n, float alpha, bool relu,
                                  uint32_t block_dim, hipStream_t stream) {
  if (m < 0 || k < 0 || n < 0) return invalid("matmul_add_leakyrelu: negative extent");
  if (m == 0 || n == 0) return ok_status();
  if (!out) return invalid("matmul_add_leakyrelu: null tensor pointer");   // a null bias means "no bias"
  if (k > 0 && (!a || !b)) return invalid("matmul_add_leakyrelu: null input matrix");
  if (m > 0x7fffffff || n > 0x7fffffff || k > 0x7fffffff)
    return invalid("matmul_add_leakyrelu: extent exceeds 2^31-1");
  if ((m * n) / n != m || m * n > INT64_MAX / 4 || (k && (m * k > INT64_MAX / 4 || k * n > INT64_MAX / 4)))
    return invalid("matmul_add_leakyrelu: extent overflow");

  const bool al = aligned16(a) && aligned16(b) && aligned16(out) &&
                  ((reinterpret_cast<uintptr_t>(bias) & (F16IO ? 15u : 7u)) == 0);
  // 256 x 256 tiles for fewer than half of the CUs: 128 x 128 tiles keep four times as many busy
  // (2048^3: 240 -> 390 TFLOP/s; at 3072^3, 144 tiles, the large ones are still faster)
  const bool few_big_tiles = (m / 256) * (n / 256) < (int64_t)device_cus() / 2 && m % 128 == 0 && n % 128 == 0;
  if (al && !few_big_tiles && matmul_dma_supported(m, k, n)) {
    if constexpr (F16IO)
      return launch_matmul_dma_f16(a, b, static_cast<const float *>(bias), static_cast<float *>(out),
                                   (int)m, (int)k, (int)n, alpha, relu, block_dim, stream);
    else
      return launch_matmul_dma(a, b, static_cast<const uint16_t *>(bias), static_cast<uint16_t *>(out),
                               (int)m, (int)k, (int)n, alpha, relu, block_dim, stream);
  }
  // A row count that is no multiple of 256 over shapes the direct-to-LDS kernel otherwise takes
  // (rows are what varies in practice: a batch, a sequence): the whole tiles on that kernel and
  // the last m % 256 rows in a launch of their own on the bounds-checked kernel below, instead
  // of everything on the latter (8200 x 8192 x 8192: 680 -> 1400 TFLOP/s).  The two launches
  // write disjoint rows.
  const int64_t m_whole = m - m % 256;
  if (al && !block_dim && m_whole < m && matmul_dma_supported(256, k, n) &&
      (m_whole / 256) * (n / 256) >= (int64_t)device_cus() / 2) {
    const LaunchStatus whole = launch_matmul_any_io<F16IO>(a, b, bias, out, m_whole, k, n, alpha, relu, 0, stream);
    if (whole.code != 0) return whole;
    const int64_t out_bytes = F16IO ? 4 : 2;
    return launch_matmul_any_io<F16IO>(a + m_whole * k, b, bias, static_cast<char *>(out) + m_whole * n * out_bytes, m - m_whole,
                                       k, n, alpha, relu, 0, stream);
  }
  if (al && !few_big_tiles && k >= kBK && k % kBK == 0 && m % 256 == 0 && n % 256 == 0)
    return launch_mfma<2, 4, 4, 2, F16IO>(a, b, bias, out, (int)m, (int)k, (int)n, alpha, relu, block_dim, stream);
  if (al && k >= kBK && k % kBK == 0 && m % 128 == 0 && n % 128 == 0)
    return launch_mfma<2, 2, 2, 2, F16IO>(a, b, bias, out, (int)m, (int)k, (int)n, alpha, relu, block_dim, stream);
  // any M, K and N multiples of 8 (every row starts on a 16-byte boundary): the same kernel, bounds-checked
  if (al && k >= 8 && k % 8 == 0 && n % 8 == 0 && (int64_t)((m + 127) / 128) * ((n + 127) / 128) <= 0x7fffffff)
    return launch_mfma<2, 2, 2, 2, F16IO, 1>(a, b, bias, out, (int)m, (int)k, (int)n, alpha, relu, block_dim, stream);
  // anything else that is not tiny: element accesses into the same MFMA loop
  if (k >= 1 && m * n >= 128 * 128 && (int64_t)((m + 127) / 128) * ((n + 127) / 128) <= 0x7fffffff)
    return launch_mfma<2, 2, 2, 2, F16IO, 2>(a, b, bias, out, (int)m, (int)k, (int)n, alpha, relu, block_dim, stream);

  const int tiles_m = (int)((m + 15) / 16), tiles_n = (int)((n + 15) / 16);
  int64_t blocks = (int64_t)tiles_m * tiles_n;
  if (block_dim) blocks = block_dim;
  if (blocks > 0x7fffffff) blocks = 0x7fffffff;
  AFIR_LAUNCH("matmul_bias_leakyrelu_any<F16IO>", matmul_bias_leakyrelu_any<F16IO>, dim3((unsigned)blocks), dim3(256), 0, stream,
                     a, b, bias, out, (int)m, (int)k, (int)n, alpha, relu ? 1 : 0, tiles_m, tiles_n);
  return after_launch();
}

}  // namespace

LaunchStatus launch_matmul_add_leakyrelu(const uint16_t *a, const uint16_t *b,
                                         const uint16_t *bias, uint16_t *out, int64_t m,
                                         int64_t k, int64_t n, float alpha, bool relu,
                                         uint32_t block_dim, hipStream_t stream) {
  return launch_matmul_any_io<false>(a, b, bias, out, m, k, n, alpha, relu, block_dim, stream);
}

LaunchStatus launch_matmul_add_leakyrelu_f16(const uint16_t *a, const uint16_t *b, const float *bias,
                                             float *out, int64_t m, int64_t k, int64_t n,
                                             float alpha, bool relu, uint32_t block_dim,
                                             hipStream_t stream) {
  return launch_matmul_any_io<true>(a, b, bias, out, m, k, n, alpha, relu, block_dim, stream);
}

}  // namespace afir
