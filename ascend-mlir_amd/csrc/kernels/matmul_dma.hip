// Matmul + bias + leaky relu for large, tile-aligned shapes (M, N multiples of
// 256, K a multiple of 64): the MFMA-bound fast path.
//
// The feed is the bottleneck of a bf16 GEMM on this chip: one K step of 32 is
// ~0.4 us of MFMA work per CU while a global load takes ~2 us to come back
// under load, so several K steps have to be in flight.  Registers cannot hold
// them, LDS can: tiles are copied global -> LDS directly (global_load_lds, 16
// bytes per lane, no VGPR staging) into two rings that together fill the
// 160 KiB of LDS:
//
//   A ring: 3 slots of [256 m][64 k] bf16 (128-byte rows, 32 KiB): 64 k at a
//           time so that every row segment is a full 128-byte line -- with
//           64-byte segments the feed alone took 30 % longer;
//   B ring: 4 slots of [32 k][256 n] bf16 (512-byte rows, 16 KiB).
//
// A direct-to-LDS load writes lane l's 16 bytes at base + 16*l, so a wave
// fills 1 KiB of contiguous LDS; which 16-byte chunk of global memory a lane
// fetches is free, and that is where the bank swizzle goes:
//   A: chunk c of row r lands at chunk position c ^ ((r>>1)&7);
//   B: chunk c of row k lands at chunk position c ^ ((k&3)<<2).
// The A operand of an MFMA is one 128-bit LDS read per lane (8 consecutive k
// of one m).  The B operand needs 8 consecutive k of one n from a tile whose
// rows run along n: ds_read_b64_tr_b16 does that transpose in the LDS unit
// (within 16 lanes, lanes 4r..4r+3 address row r, lane i receives column i of
// the four rows).  With the swizzles above both reads are bank-conflict free.
//
// The compiler cannot be trusted to wait for exactly the right stage (it
// drains every outstanding direct-to-LDS load before any LDS read that might
// alias one), so the operand reads are issued from inline asm and the waits
// are explicit: s_waitcnt vmcnt(n) + s_barrier once per K step of 32, which
// leaves the two youngest B stages and the youngest A slice in flight.
// Operand reads are software-pipelined one k16 substep ahead of the MFMAs.
//
// Every tile starts its walk over K at a different offset and wraps around
// (K-stagger): the row pitch of A and B is a large power of two, so without it
// all workgroups of the chip ask the same few L2 / memory channels for the
// same K offset at the same time.
//
// 8 waves as 2(m) x 4(n), wave tile 128 x 64 = 4 x 2 MFMA tiles of 32x32,
// v_mfma_f32_32x32x16_bf16 with the operands swapped (B as the row operand) so
// that a lane holds four consecutive n of one m for the fused epilogue.
// (AFIR_MM_WAVES_N=2 builds 4 waves of 128 x 128 instead: a third fewer LDS
// operand bytes per MFMA, but one wave per SIMD leaves the matrix unit idle
// around every barrier; measured on MI355X it is 11 % slower on constant
// operands and equal, within 1 %, on N(0, 1/sqrt(K)) operands, where the board
// power limit sets the pace.)
#include <type_traits>

#include "kernels.h"

namespace afir {

namespace {

#ifndef AFIR_MM_KSTAGGER_M
#define AFIR_MM_KSTAGGER_M 2
#endif
#ifndef AFIR_MM_KSTAGGER_N
#define AFIR_MM_KSTAGGER_N 1
#endif
// Measurement builds only (the benchmark's probe library compiles this file again with
// -DAFIR_MM_ABLATE=1 or 2 under another namespace name): 1 leaves the global -> LDS feed
// out of the K loop after the prologue, 2 the LDS operand reads as well, so that what
// remains can be timed on its own.  Such a build computes nothing meaningful.
#ifndef AFIR_MM_ABLATE
#define AFIR_MM_ABLATE 0
#endif
constexpr int kBK = 32;                   // K per B stage
constexpr int kBM = 256, kBN = 256;
constexpr int kASlots = 3, kBSlots = 4;
constexpr int kSlotA = kBM * 64 * 2;      // 32 KiB: 64 k per A slice
constexpr int kSlotB = kBK * kBN * 2;     // 16 KiB
constexpr int kRingB = kASlots * kSlotA;  // byte offset of the B ring
constexpr int kLdsBytes = kASlots * kSlotA + kBSlots * kSlotB;  // 160 KiB

typedef __attribute__((address_space(3))) unsigned char lds_byte;
typedef __attribute__((address_space(3))) void lds_void;
typedef __attribute__((address_space(1))) const void gbl_void;

__device__ __forceinline__ void map_tile_dma(int p, int tiles_m, int tiles_n, int &tm, int &tn) {
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

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// Operands of one k16 substep: TMW A fragments (m tiles, 4 KiB apart) and TNW
// B fragments (n tiles, each two transposing 64-bit reads 4 rows apart).
// issue_reads only issues; the registers must not be touched until
// settle_reads, which waits for the LDS unit and hands the same registers back
// as fresh values.
template <int TMW, int TNW>
struct Operands {
  u32x4 a[TMW];
  u32x2 b[TNW][2];
};

template <int OFF>
__device__ __forceinline__ void read_a(uint32_t addr, u32x4 &dst) {
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=&v"(dst) : "v"(addr), "n"(OFF) : "memory");
}
template <int OFF>
__device__ __forceinline__ void read_b(uint32_t addr, u32x2 &dst) {
  asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=&v"(dst) : "v"(addr), "n"(OFF) : "memory");
}

template <int KS, int TMW, int TNW>  // KS: k16 substep within the B stage (0 or 1)
__device__ __forceinline__ void issue_reads(uint32_t a_addr, const uint32_t (&b_addr)[TNW],
                                            Operands<TMW, TNW> &o) {
  constexpr int kOff = KS * 16 * 512;  // 16 rows of B
  read_a<0>(a_addr, o.a[0]);
  read_a<4096>(a_addr, o.a[1]);
  if constexpr (TMW == 4) {
    read_a<8192>(a_addr, o.a[2]);
    read_a<12288>(a_addr, o.a[3]);
  }
#pragma unroll
  for (int j = 0; j < TNW; ++j) {
    read_b<kOff>(b_addr[j], o.b[j][0]);
    read_b<kOff + 4 * 512>(b_addr[j], o.b[j][1]);
  }
}

template <int TMW, int TNW>
__device__ __forceinline__ void settle_reads(Operands<TMW, TNW> &o) {
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  // volatile asm statements keep their order: every register counts as
  // rewritten after the wait, so no use can move above it
#pragma unroll
  for (int i = 0; i < TMW; ++i) asm volatile("" : "+v"(o.a[i]));
#pragma unroll
  for (int j = 0; j < TNW; ++j) {
    asm volatile("" : "+v"(o.b[j][0]));
    asm volatile("" : "+v"(o.b[j][1]));
  }
}

struct Par0 { static constexpr int value = 0; };
struct Par1 { static constexpr int value = 1; };
struct Steady { static constexpr bool value = true; };
struct Drain { static constexpr bool value = false; };

// WM x WN waves (m x n), wave tile (256/WM) x (256/WN): 2 x 4 waves of
// 128 x 64, or 2 x 2 waves of 128 x 128 (one wave per SIMD, two thirds of the
// LDS operand bytes per MFMA).
//
// F16IO = false: A, B, bias, out are bf16.  F16IO = true: A, B are f16, bias and
// out are float32 (the types of the reference's own matmul example,
// examples/matmul-add-leakyrelu/step0_input.mlir:10-15): the same rings and
// reads (both element types are 16 bits wide), the f16 MFMA, and an epilogue
// that stores the float32 value unrounded.
template <int WM, int WN, bool F16IO>
__global__ __launch_bounds__(WM * WN * 64) void matmul_bias_leakyrelu_dma(
    const uint16_t *__restrict__ A, const uint16_t *__restrict__ B,
    const void *__restrict__ bias_v, void *__restrict__ out_v, int M, int K, int N,
    float alpha, int relu, int tiles_m, int tiles_n) {
  extern __shared__ __align__(1024) unsigned char smem[];
  lds_byte *const lds = (lds_byte *)smem;
  const uint32_t lds_base = (uint32_t)(uintptr_t)lds;

  const int t = threadIdx.x, lane = t & 63;
  constexpr int TMW = 8 / WM;            // 32-row MFMA tiles per wave along m
  constexpr int TNW = 8 / WN;            // 32-column MFMA tiles per wave along n
  constexpr int NWAVES = WM * WN;
  constexpr int A_REG = 32 / NWAVES;     // 1 KiB direct-to-LDS regions per wave per A slice
  constexpr int B_REG = 16 / NWAVES;     // ... per B stage
  constexpr int kSteadyVm = 2 * B_REG + A_REG;  // loads younger than what the next stage needs
  const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const int wm = wave / WN, wn = wave % WN;
  const int KT = K / kBK;   // B stages; even, the launcher requires K % 64 == 0
  const int KT2 = KT >> 1;  // A slices

  // ---- per-lane operand read addresses, relative to a ring slot ----
  const int lrow = lane & 31, lk = lane >> 5;
  // substep ks (0..3) of the slice reads chunk 2*ks + lk:  a_rd ^ (ks * 32)
  const uint32_t a_rd =
      (uint32_t)((wm * TMW * 32 + lrow) * 128 + (lk ^ ((lrow >> 1) & 7)) * 16);
  const int g = lane >> 4, li = lane & 15;
  uint32_t b_rd[TNW];
#pragma unroll
  for (int j = 0; j < TNW; ++j) {
    const int ntile = wn * TNW + j;
    const int c16 = ntile * 4 + (g & 1) * 2 + ((li & 3) >> 1);
    const int phys = c16 ^ ((li >> 2) << 2);
    b_rd[j] = (uint32_t)(kRingB + ((g >> 1) * 8 + (li >> 2)) * 512 + phys * 16 + (li & 1) * 8);
  }

  for (int p = blockIdx.x; p < tiles_m * tiles_n; p += gridDim.x) {
    int tile_m, tile_n;
    map_tile_dma(p, tiles_m, tiles_n, tile_m, tile_n);
    const int m0 = tile_m * kBM, n0 = tile_n * kBN;

    // K-stagger: this tile walks stages kfirst, kfirst+1, ..., wrapping at KT.
    // kfirst is even so that A slices (two stages) stay aligned.
    const int kfirst =
        (int)(((unsigned)(tile_m * AFIR_MM_KSTAGGER_M + tile_n * AFIR_MM_KSTAGGER_N) * 2u) %
              (unsigned)KT);

    // ---- per-lane global sources of the direct-to-LDS loads ----
    // A slice: 32 regions of 1 KiB (8 rows x 128 B), A_REG per wave.
    // B stage: 16 regions of 1 KiB (2 rows x 512 B), B_REG per wave.
    const uint16_t *ga[A_REG], *gb[B_REG];
#pragma unroll
    for (int q = 0; q < A_REG; ++q) {
      const int arow = (wave * A_REG + q) * 8 + (lane >> 3);
      const int ac = (lane & 7) ^ ((arow >> 1) & 7);
      ga[q] = A + (int64_t)(m0 + arow) * K + ac * 8 + (int64_t)kfirst * kBK;
    }
#pragma unroll
    for (int q = 0; q < B_REG; ++q) {
      const int bk = (wave * B_REG + q) * 2 + (lane >> 5);
      const int bc = (lane & 31) ^ ((bk & 3) << 2);
      gb[q] = B + (int64_t)(bk + kfirst * kBK) * N + n0 + bc * 8;
    }
    int ka_next = kfirst >> 1;  // slice (64 k) the next A issue fetches
    int kb_next = kfirst;       // stage (32 k) the next B issue fetches

    auto issue_a = [&](int slot) {
      lds_byte *dst = lds + slot * kSlotA + wave * (A_REG * 1024);
#pragma unroll
      for (int q = 0; q < A_REG; ++q)
        __builtin_amdgcn_global_load_lds((gbl_void *)ga[q], (lds_void *)(dst + q * 1024), 16, 0, 0);
      ka_next = (ka_next + 1 == KT2) ? 0 : ka_next + 1;
      const int64_t step = (ka_next == 0) ? -(int64_t)(KT2 - 1) * 64 : (int64_t)64;
#pragma unroll
      for (int q = 0; q < A_REG; ++q) ga[q] += step;
    };
    auto issue_b = [&](int slot) {
      lds_byte *dst = lds + kRingB + slot * kSlotB + wave * (B_REG * 1024);
#pragma unroll
      for (int q = 0; q < B_REG; ++q)
        __builtin_amdgcn_global_load_lds((gbl_void *)gb[q], (lds_void *)(dst + q * 1024), 16, 0, 0);
      kb_next = (kb_next + 1 == KT) ? 0 : kb_next + 1;
      const int64_t step = (kb_next == 0) ? -(int64_t)(KT - 1) * kBK * N : (int64_t)kBK * N;
#pragma unroll
      for (int q = 0; q < B_REG; ++q) gb[q] += step;
    };

    f32x16 acc[TMW][TNW];
#pragma unroll
    for (int i = 0; i < TMW; ++i)
#pragma unroll
      for (int j = 0; j < TNW; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

    auto multiply = [&](const Operands<TMW, TNW> &o) {
#pragma unroll
      for (int j = 0; j < TNW; ++j) {
        const u32x4 bw = {o.b[j][0].x, o.b[j][0].y, o.b[j][1].x, o.b[j][1].y};
#pragma unroll
        for (int i = 0; i < TMW; ++i) {
          if constexpr (F16IO)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(
                __builtin_bit_cast(f16x8, bw), __builtin_bit_cast(f16x8, o.a[i]), acc[i][j], 0, 0, 0);
          else
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                __builtin_bit_cast(bf16x8, bw), __builtin_bit_cast(bf16x8, o.a[i]), acc[i][j], 0, 0,
                0);
        }
      }
    };
    // operand reads for a stage held in A slot sa / B slot sbk; the stage is the
    // first (par 0) or second (par 1) half of its A slice; h = k16 substep
    auto reads = [&](int sa, int sbk, int par, int h, Operands<TMW, TNW> &o, bool prologue = false) {
      if (AFIR_MM_ABLATE >= 2 && !prologue) return;
      const uint32_t aa =
          lds_base + (uint32_t)(sa * kSlotA) + (a_rd ^ (uint32_t)((par * 2 + h) * 32));
      const uint32_t bb = lds_base + (uint32_t)(sbk * kSlotB);
      uint32_t ba[TNW];
#pragma unroll
      for (int j = 0; j < TNW; ++j) ba[j] = bb + b_rd[j];
      if (h == 0)
        issue_reads<0>(aa, ba, o);
      else
        issue_reads<1>(aa, ba, o);
    };

    // prologue (the launcher guarantees KT >= 8): fill both rings, oldest first
    issue_a(0);
    issue_b(0);
    issue_b(1);
    issue_a(1);
    issue_b(2);
    issue_b(3);
    issue_a(2);
    wait_vmcnt<3 * B_REG + 2 * A_REG>();  // everything younger than A(0), B(0)
    __builtin_amdgcn_s_barrier();
    Operands<TMW, TNW> even, odd;
    reads(0, 0, 0, 0, even, true);
    settle_reads(even);
    if (AFIR_MM_ABLATE >= 2) odd = even;

    // One step of the pipeline for stage s of parity PAR:
    //   reads(s, substep 1) in flight | MFMAs(s, substep 0)
    //   wait until stage s+1 has landed, barrier: everyone is done reading s
    //   reads(s+1, substep 0) in flight, refill the freed slots | MFMAs(s, substep 1)
    // Refill after stage s: B(s+4) into s's B slot; after an odd s also the A
    // slice (s+5)/2 into the slot of the slice just finished.  In the steady
    // state both exist and the vmcnt is exact: younger than what stage s+1 needs
    // are exactly 2 B stages and 1 A slice.  Otherwise drain.
    int sa = 0, sb = 0;  // ring slots of the stage being multiplied
    auto step = [&](auto par_tag, auto mode_tag, bool has_next, bool refill_b, bool refill_a) {
      constexpr int PAR = decltype(par_tag)::value;
      constexpr bool STEADY = decltype(mode_tag)::value;
      const int sb_next = (sb + 1 == kBSlots) ? 0 : sb + 1;
      const int sa_next = PAR ? ((sa + 1 == kASlots) ? 0 : sa + 1) : sa;
      reads(sa, sb, PAR, 1, odd);
      __builtin_amdgcn_sched_barrier(0);
      multiply(even);
      __builtin_amdgcn_sched_barrier(0);
      settle_reads(odd);
      if (STEADY || has_next) {
        if (STEADY)
          wait_vmcnt<kSteadyVm>();
        else
          wait_vmcnt<0>();
        __builtin_amdgcn_s_barrier();
        reads(sa_next, sb_next, PAR ^ 1, 0, even);
        if (AFIR_MM_ABLATE == 0) {
          if (PAR && (STEADY || refill_a)) issue_a(sa);
          if (STEADY || refill_b) issue_b(sb);
        }
      }
      multiply(odd);
      __builtin_amdgcn_sched_barrier(0);
      if (STEADY || has_next) settle_reads(even);
      sa = sa_next;
      sb = sb_next;
    };

    int s = 0;
    for (; s + 6 < KT; s += 2) {  // both refills exist: B(s+4), B(s+5), A((s+6)/2)
      step(Par0{}, Steady{}, true, true, true);
      step(Par1{}, Steady{}, true, true, true);
    }
    for (; s < KT; s += 2) {
      step(Par0{}, Drain{}, true, s + 4 < KT, false);
      step(Par1{}, Drain{}, s + 2 < KT, s + 5 < KT, s + 6 < KT);
    }

    // Epilogue.  A lane holds m = lane%32, n = 8q + 4*(lane/32) + e of each
    // 32x32 block, i.e. 8 bytes (bf16) or 16 bytes (float32) of an output row
    // per store: written straight to memory that is a fraction of a line per row
    // per instruction, and the partial lines of the bf16 form cost three times
    // the write traffic.  So each wave stages 32 rows of its tile (64 n = one
    // or two 128-byte lines per row) in LDS and stores them as full lines,
    // eight or four rows per instruction.  The rings are free once every wave
    // has left the K loop; a wave's 4 or 8 KiB staging area is private, and
    // the LDS unit keeps a wave's accesses in order, so no further barrier is
    // needed until the next tile refills the rings.  The 16-byte chunk column
    // is XOR-ed with a function of the row: conflict-free for the 8- or
    // 16-byte writes (32 rows x 2 halves) and for the 16-byte row reads.
    __builtin_amdgcn_s_barrier();
    {
      constexpr int kOutBytes = F16IO ? 4 : 2;
      constexpr int CH = TNW * 32 * kOutBytes / 16;   // 16-byte chunks per staged row
      constexpr int kRowBytes = CH * 16;       // 128 .. 512
      constexpr int kRowsPerPass = 64 / CH;    // rows one store instruction covers
      unsigned char *const stage = smem + wave * (32 * kRowBytes);
      const int lm = lane & 31, lq = lane >> 5;
      const int rr = lane / CH, cc = lane % CH;
      // two 128-byte rows share a swizzle value (they span the same banks as
      // one 256-byte row)
      auto swz = [](int r) { return CH == 8 ? ((r >> 1) & 7) : (r & (CH - 1)); };
      typedef typename std::conditional<F16IO, f32x4, u32x2>::type BiasRaw;
      BiasRaw braw[TNW][4];
#pragma unroll
      for (int j = 0; j < TNW; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int n = n0 + (wn * TNW + j) * 32 + 8 * q + 4 * lq;
          // no bias: -0, the identity of the add
          if constexpr (F16IO)
            braw[j][q] = bias_v ? *reinterpret_cast<const f32x4 *>(static_cast<const float *>(bias_v) + n)
                                : f32x4{-0.f, -0.f, -0.f, -0.f};
          else
            braw[j][q] = bias_v ? *reinterpret_cast<const u32x2 *>(static_cast<const uint16_t *>(bias_v) + n)
                                : u32x2{0x80008000u, 0x80008000u};
        }
#pragma unroll
      for (int i = 0; i < TMW; ++i) {
#pragma unroll
        for (int j = 0; j < TNW; ++j) {
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            float b0, b1, b2, b3;
            if constexpr (F16IO) {
              b0 = braw[j][q][0]; b1 = braw[j][q][1]; b2 = braw[j][q][2]; b3 = braw[j][q][3];
            } else {
              b0 = bf16_lo(braw[j][q].x); b1 = bf16_hi(braw[j][q].x);
              b2 = bf16_lo(braw[j][q].y); b3 = bf16_hi(braw[j][q].y);
            }
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
              const int chunk = (j * 8 + q * 2 + lq) ^ swz(lm);
              *reinterpret_cast<f32x4 *>(stage + lm * kRowBytes + chunk * 16) = w;
            } else {
              u32x2 w;
              w.x = pack_bf16(v0, v1);
              w.y = pack_bf16(v2, v3);
              const int chunk = (j * 4 + q) ^ swz(lm);
              *reinterpret_cast<u32x2 *>(stage + lm * kRowBytes + chunk * 16 + lq * 8) = w;
            }
          }
        }
#pragma unroll
        for (int tq = 0; tq < 32 / kRowsPerPass; ++tq) {
          const int r = rr + kRowsPerPass * tq;
          const u32x4 line =
              *reinterpret_cast<const u32x4 *>(stage + r * kRowBytes + ((cc ^ swz(r)) * 16));
          const int m = m0 + (wm * TMW + i) * 32 + r;
          unsigned char *const row = static_cast<unsigned char *>(out_v) +
                                     ((int64_t)m * N + n0 + wn * (TNW * 32)) * kOutBytes;
          *reinterpret_cast<u32x4 *>(row + cc * 16) = line;
        }
      }
    }
    // every wave must be done reading the rings before the next tile refills them
    __builtin_amdgcn_s_barrier();
  }
}

}  // namespace

bool matmul_dma_supported(int64_t m, int64_t k, int64_t n) {
  return m % kBM == 0 && n % kBN == 0 && k % 64 == 0 && k >= 8 * kBK;
}

#ifndef AFIR_MM_WAVES_M
#define AFIR_MM_WAVES_M 2
#endif
#ifndef AFIR_MM_WAVES_N
#define AFIR_MM_WAVES_N 4
#endif
#ifndef AFIR_MM_GRID
#define AFIR_MM_GRID kNumCU
#endif

namespace {

template <bool F16IO>
LaunchStatus launch_dma(const uint16_t *a, const uint16_t *b, const void *bias, void *out, int m,
                        int k, int n, float alpha, bool relu, uint32_t block_dim,
                        hipStream_t stream) {
  constexpr int WM = AFIR_MM_WAVES_M, WN = AFIR_MM_WAVES_N;
  auto kernel = matmul_bias_leakyrelu_dma<WM, WN, F16IO>;
  static hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                               hipFuncAttributeMaxDynamicSharedMemorySize,
                                               kLdsBytes);
  if (attr != hipSuccess) return LaunchStatus{2u, hipGetErrorString(attr)};
  const int tiles_m = m / kBM, tiles_n = n / kBN;
  // One workgroup fills a CU's LDS, so the grid is persistent: one workgroup
  // per CU, each walking its share of the tiles.
  int64_t blocks = (int64_t)tiles_m * tiles_n;
  if (blocks > AFIR_MM_GRID) blocks = AFIR_MM_GRID;
  if (block_dim) blocks = block_dim;
  hipLaunchKernelGGL(kernel, dim3((unsigned)blocks), dim3(WM * WN * 64), kLdsBytes, stream, a, b,
                     bias, out, m, k, n, alpha, relu ? 1 : 0, tiles_m, tiles_n);
  return after_launch();
}

}  // namespace

LaunchStatus launch_matmul_dma(const uint16_t *a, const uint16_t *b, const uint16_t *bias,
                               uint16_t *out, int m, int k, int n, float alpha, bool relu,
                               uint32_t block_dim, hipStream_t stream) {
  return launch_dma<false>(a, b, bias, out, m, k, n, alpha, relu, block_dim, stream);
}

LaunchStatus launch_matmul_dma_f16(const uint16_t *a, const uint16_t *b, const float *bias,
                                   float *out, int m, int k, int n, float alpha, bool relu,
                                   uint32_t block_dim, hipStream_t stream) {
  return launch_dma<true>(a, b, bias, out, m, k, n, alpha, relu, block_dim, stream);
}

}  // namespace afir
