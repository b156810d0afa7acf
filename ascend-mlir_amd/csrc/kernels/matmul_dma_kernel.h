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
//   B: chunk c of row k lands at chunk position c ^ ((k&3)<<2) ^ (((k>>3)&1)<<1).
//
// The matrix instruction is v_mfma_f32_16x16x32_bf16: K = 32 per instruction,
// a lane holds 8 consecutive k of one row (A) or one column (B), 4 accumulator
// registers per 16 x 16 tile.  It was chosen over v_mfma_f32_32x32x16_bf16 by
// measurement: the chip runs this kernel against its board power limit, and
// on operands drawn from N(0, 1/sqrt(K)) a register-only loop of the 16x16x32
// form sustains 2040 TFLOP/s where the 32x32x16 form sustains 1765 (on
// constant operands both reach 2470): per flop the accumulators are read and
// written half as often.
// The A operand of an MFMA is one 128-bit LDS read per lane.  The B operand
// needs 8 consecutive k of one n from a tile whose rows run along n:
// ds_read_b64_tr_b16 does that transpose in the LDS unit (within 16 lanes,
// lanes 4r..4r+3 address row r, lane i receives column i of the four rows),
// two of them four rows apart per operand.  With the swizzles above both
// reads are bank-conflict free.
//
// The compiler cannot be trusted to wait for exactly the right stage (it
// drains every outstanding direct-to-LDS load before any LDS read that might
// alias one), so the operand reads and the direct-to-LDS loads are issued from
// inline asm and the waits are explicit: s_waitcnt vmcnt(n) + s_barrier once
// per K step of 32, which leaves the two youngest B stages and the youngest A
// slice in flight.
//
// The K loop is ONE instruction stream per wave in which every operand read
// and every direct-to-LDS load sits behind an MFMA (pinned with scheduling
// barriers).  All eight waves pass the workgroup barrier together, so a block
// of reads or loads issued after it would leave the matrix units of all four
// SIMDs idle at the same time; behind an MFMA, which occupies the unit for 16
// cycles, an instruction issues for free.  The reads go behind the first MFMAs
// of a phase so that the remaining ones cover their latency.  The direct-to-LDS
// loads take a scalar base (tile, region, K position) plus a 32-bit per-lane
// offset, so the loop spends no vector registers or instructions on addresses.
// Measured on MI355X, 8192^3, TFLOP/s on constant / N(0, 1/sqrt(K)) operands:
// 32x32x16 MFMAs with reads and loads in blocks 1630 / 1235; 16x16x32 in blocks
// 1565 / 1320; 16x16x32 interleaved as described 1700 / 1350-1365 (the vendor
// GEMM without the epilogue, same runs: 1775 / 1360-1385).
//
// What the loop then waits for is the memory system behind the loads: with every
// load pointed at the same 1 KiB (issue and LDS-write cost only) the kernel runs
// 2095 / 1600, with real addresses 1770 / 1385.  A stage has only as long to
// arrive as the rings are deep, so the refills go out as early as the barrier
// allows (the B stage right behind the barrier of the step that frees its slot:
// 1875 / 1455), and between tiles nothing drains: the first stages of the next
// tile are requested during the epilogue (per-tile overhead 13 -> 6.5 us of 250).
//
// Every tile starts its walk over K at a different offset and wraps around
// (K-stagger): the row pitch of A and B is a large power of two, so without it
// all workgroups of the chip ask the same few L2 / memory channels for the
// same K offset at the same time.
//
// 8 waves as 2(m) x 4(n), two per SIMD (one wave per SIMD cannot issue 16-cycle
// MFMAs back to back: 1815 of 2470 TFLOP/s in a register-only loop); wave tile
// 128 x 64 = 8 x 4 MFMA tiles of 16 x 16, with the operands swapped (B as the
// row operand) so that a lane holds four consecutive n of one m for the fused
// epilogue.
#pragma once

#include <type_traits>

#include "kernels.h"

namespace afir {

namespace dma {

// Compile-time choices a tile search can vary (bin/autotuner, parameters build_<MACRO>;
// ascend-mlir_amd/examples/autotune-matmul): the K offsets tiles start from, and how many
// tile rows an XCD's 32 workgroups cover at once (their patch is GROUP_M x 32 / GROUP_M tiles).
#ifndef AFIR_MM_GROUP_M
#define AFIR_MM_GROUP_M 4
#endif
#ifndef AFIR_MM_KSTAGGER_M
#define AFIR_MM_KSTAGGER_M 1
#endif
#ifndef AFIR_MM_KSTAGGER_N
#define AFIR_MM_KSTAGGER_N 0
#endif
// What an instance of the kernel does with its operand feed.  The library instantiates the
// kernel with FullFeed only; a measurement build may instantiate it with a policy of its own
// that leaves parts of the K loop out or redirects the loads, to time what remains.
struct FullFeed {
  static constexpr bool kLoads = true;          // global -> LDS loads in the K loop (the ring fills before it always run)
  static constexpr bool kOperandReads = true;   // LDS -> register operand reads in the K loop
  static constexpr int kWrapStages = 0;         // > 0: the walk over K wraps after this many stages of 32 (even)
  // the source of one direct-to-LDS load: wave-uniform base + per-lane byte offset
  __device__ static void source(const char *&, uint32_t &, const void *, int) {}
};

// MFMAs between two refill loads of a phase (1: back to back; 2 measured 0.5 % faster)
// 1: the B stage that a step frees is refilled in that step's second phase, right after the
// barrier, instead of in the next step's first phase (0).  A B stage then has 3 steps to
// arrive instead of 2.2: 1400 -> 1455 TFLOP/s on the workload's operands, 1770 -> 1875 on
// constants.  (The same move for the A slice, six loads in one phase beside its twelve operand
// reads, measured 6 % slower: the reads come back late.)
#ifndef AFIR_MM_B_EARLY
#define AFIR_MM_B_EARLY 1
#endif
// the output rows leave with non-temporal stores: a tile's 128 KiB times 32 workgroups is the
// whole L2 of an XCD, and written through it they evict the A / B lines the next tile reads
// (1444 -> 1456 TFLOP/s)
#ifndef AFIR_MM_NT_STORE
#define AFIR_MM_NT_STORE 1
#endif
// the order of a phase's sixteen MFMAs: 0 walks the four m tiles under one n tile (consecutive
// instructions share the B fragment), 1 the four n tiles under one m tile (they share the A one)
#ifndef AFIR_MM_MFMA_A_OUTER
#define AFIR_MM_MFMA_A_OUTER 0
#endif
#ifndef AFIR_MM_DMA_STRIDE
#define AFIR_MM_DMA_STRIDE 2
#endif
constexpr int kBK = 32;                   // K per B stage
constexpr int kBM = 256, kBN = 256;
constexpr int kASlots = 3, kBSlots = 4;
constexpr int kSlotA = kBM * 64 * 2;      // 32 KiB: 64 k per A slice
constexpr int kSlotB = kBK * kBN * 2;     // 16 KiB
constexpr int kRingB = kASlots * kSlotA;  // byte offset of the B ring
constexpr int kLdsBytes = kASlots * kSlotA + kBSlots * kSlotB;  // 160 KiB

constexpr int kWavesM = 2, kWavesN = 4, kWaves = kWavesM * kWavesN;
constexpr int kTM = kBM / kWavesM / 16;   // 8: 16-row MFMA tiles per wave along m
constexpr int kTN = kBN / kWavesN / 16;   // 4: 16-column MFMA tiles per wave along n
// The first kFeedWaves waves of a workgroup issue the direct-to-LDS loads and wait for them.
// With fewer than all eight, the others never wait on a load counter of their own and can touch,
// kPrefetch stages ahead, the lines the feed will ask for (see prefetch below): a load that is
// not waited for costs no time however long it takes, and the feed then finds its lines in L2.
#ifndef AFIR_MM_FEED_WAVES
#define AFIR_MM_FEED_WAVES 8
#endif
#ifndef AFIR_MM_PREFETCH
#define AFIR_MM_PREFETCH 0
#endif
constexpr int kFeedWaves = AFIR_MM_FEED_WAVES;
constexpr int kPrefetch = AFIR_MM_PREFETCH;   // stages of 32 k the prefetch runs ahead of the multiply (0: none)
static_assert(kFeedWaves == 8 || kFeedWaves == 4, "the feed is issued by all eight waves or by the first four");
static_assert(kPrefetch == 0 || (kFeedWaves == 4 && kPrefetch % 2 == 0),
              "prefetching waves issue no feed loads; the distance is a whole number of A slices");
constexpr int kAReg = 32 / kFeedWaves;    // 1 KiB direct-to-LDS regions per feeding wave per A slice
constexpr int kBReg = 16 / kFeedWaves;    // ... per B stage
constexpr int kSteadyVm = 2 * kBReg + kAReg;  // loads younger than what the next stage needs


__device__ __forceinline__ void map_tile_dma(int p, int tiles_m, int tiles_n, int &tm, int &tn) {
  const int ntiles = tiles_m * tiles_n;
  int q = p;
  if ((ntiles % kNumXCD) == 0) q = (p % kNumXCD) * (ntiles / kNumXCD) + p / kNumXCD;
  constexpr int kGroupM = AFIR_MM_GROUP_M;
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

template <int OFF>
__device__ __forceinline__ void read_a(uint32_t addr, u32x4 &dst) {
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=&v"(dst) : "v"(addr), "n"(OFF) : "memory");
}
template <int OFF>
__device__ __forceinline__ void read_b(uint32_t addr, u32x2 &dst) {
  asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=&v"(dst) : "v"(addr), "n"(OFF) : "memory");
}

// Four A fragments: m tiles 2 KiB apart (16 rows of 128 bytes), starting at tile FIRST.
// The reads only issue; the registers must not be touched until settle().
template <int FIRST>
__device__ __forceinline__ void issue_a_reads(uint32_t addr, u32x4 (&a)[4]) {
  read_a<(FIRST + 0) * 2048>(addr, a[0]);
  read_a<(FIRST + 1) * 2048>(addr, a[1]);
  read_a<(FIRST + 2) * 2048>(addr, a[2]);
  read_a<(FIRST + 3) * 2048>(addr, a[3]);
}
// The B fragments of a stage: per n tile two transposing reads, 4 rows apart.
__device__ __forceinline__ void issue_b_reads(const uint32_t (&addr)[kTN], u32x2 (&b)[kTN][2]) {
#pragma unroll
  for (int j = 0; j < kTN; ++j) {
    read_b<0>(addr[j], b[j][0]);
    read_b<4 * 512>(addr[j], b[j][1]);
  }
}
// Waits for the LDS unit and hands the registers back as fresh values: volatile asm
// statements keep their order, so no use can move above the wait.
__device__ __forceinline__ void settle_wait() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }
__device__ __forceinline__ void settle(u32x4 (&a)[4]) {
#pragma unroll
  for (int i = 0; i < 4; ++i) asm volatile("" : "+v"(a[i]));
}
__device__ __forceinline__ void settle(u32x2 (&b)[kTN][2]) {
#pragma unroll
  for (int j = 0; j < kTN; ++j) {
    asm volatile("" : "+v"(b[j][0]));
    asm volatile("" : "+v"(b[j][1]));
  }
}

template <int I, int N, typename F>
__device__ __forceinline__ void static_for(F &&f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>{});
    static_for<I + 1, N>(f);
  }
}

struct Par0 { static constexpr int value = 0; };
struct Par1 { static constexpr int value = 1; };
struct Steady { static constexpr bool value = true; };
struct Drain { static constexpr bool value = false; };

// F16IO = false: A, B, bias, out are bf16.  F16IO = true: A, B are f16, bias and
// out are float32 (the types of the reference's own matmul example,
// examples/matmul-add-leakyrelu/step0_input.mlir:10-15): the same rings and
// reads (both element types are 16 bits wide), the f16 MFMA, and an epilogue
// that stores the float32 value unrounded.
// Batched = true: `M` rows are a stack of independent products of tiles_m_batch tile rows each
// (A [batch, m, K] and out [batch, m, N] densely packed are one tall matrix each; only B changes
// with the batch: b_batch_stride elements further on per batch).  The bias is shared.
template <bool F16IO, typename Feed, bool Batched = false>
__global__ __launch_bounds__(kWaves * 64) void matmul_bias_leakyrelu_dma(
    const uint16_t *__restrict__ A, const uint16_t *__restrict__ B,
    const void *__restrict__ bias_v, void *__restrict__ out_v, int M, int K, int N,
    float alpha, int relu, int tiles_m, int tiles_n, int tiles_m_batch, int64_t b_batch_stride) {
  extern __shared__ __align__(1024) unsigned char smem[];
  // (address space 3 pointers are 32 bits wide: the value is the LDS byte address)
  const uint32_t lds_base =
      (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)smem;

  const int t = threadIdx.x, lane = t & 63;
  const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const int wm = wave / kWavesN, wn = wave % kWavesN;
  const bool feeder = kFeedWaves == kWaves || wave < kFeedWaves;   // wave-uniform
  const int KT = K / kBK;   // B stages; even, the launcher requires K % 64 == 0
  // stages after which the source addresses wrap around (all of K, unless the policy says less)
  const int KW = Feed::kWrapStages > 0 && Feed::kWrapStages < KT ? Feed::kWrapStages : KT;
  const int KW2 = KW >> 1;  // ... in A slices

  // ---- per-lane operand read addresses, relative to a ring slot ----
  // A fragment of m tile i: lane reads row i*16 + lane%16, the 16-byte chunk lane/16 of the
  // stage's 64 bytes (the second stage of a slice: chunk + 4, i.e. address ^ 64)
  const int li = lane & 15, g = lane >> 4;
  const uint32_t a_rd = (uint32_t)((wm * (kTM * 16) + li) * 128 + (g ^ ((li >> 1) & 7)) * 16);
  // B fragment of n tile j: the 16-lane group g takes rows 8g .. 8g+3 (second read: +4),
  // lanes 4r .. 4r+3 of it the 32 bytes of row r that hold the tile's 16 columns
  // (n tile j: the tile's two chunks are 2j further on, and since those bits of the unswizzled
  // chunk index are zero for tile 0, the swizzled address of tile j is that of tile 0 ^ 32j)
  uint32_t b_rd0;
  {
    const int row = g * 8 + (li >> 2);
    const int c16 = (wn * kTN) * 2 + ((li & 3) >> 1);
    const int phys = c16 ^ ((row & 3) << 2) ^ (((row >> 3) & 1) << 1);
    b_rd0 = (uint32_t)(kRingB + row * 512 + phys * 16 + (li & 1) * 8);
  }

  // ---- per-lane parts of the direct-to-LDS source addresses (bytes) ----
  // An address is a wave-uniform base (tile, region, K position: scalar registers, advanced
  // with scalar arithmetic) plus a 32-bit per-lane offset that depends only on the lane and on
  // the parity of the region (row within the region, swizzled chunk), so the loads take the
  // scalar-base form and the K loop spends no vector registers or instructions on them.
  uint32_t a_lane[2], b_lane[2];
#pragma unroll
  for (int par = 0; par < 2; ++par) {
    // regions of a wave start at a multiple of kAReg * 8 rows (a multiple of 16): only the
    // parity of the region enters the swizzle
    const int arow = par * 8 + (lane >> 3);
    a_lane[par] = (uint32_t)(((int64_t)(lane >> 3) * K + ((lane & 7) ^ ((arow >> 1) & 7)) * 8) * 2);
    const int bk = (wave * kBReg + par) * 2 + (lane >> 5);
    b_lane[par] = (uint32_t)(((int64_t)(lane >> 5) * N +
                              ((lane & 31) ^ ((bk & 3) << 2) ^ (((bk >> 3) & 1) << 1)) * 8) * 2);
  }
  if (kPrefetch > 0 && !feeder) {
    // a prefetching wave issues no feed loads: the same registers hold the lane parts of its
    // own loads, one dword per lane out of 64 different 128-byte lines.  A: lane = row of a
    // 64-row quarter of the slice; B: four lines per row, 16 rows of a pair of stages.
    a_lane[0] = (uint32_t)((int64_t)lane * K * 2);
    b_lane[0] = (uint32_t)(((int64_t)(lane >> 2) * N + (lane & 3) * 64) * 2);
    a_lane[1] = 0;   // the register the loaded dwords go to; nobody reads it
  }

  // ---- state of the tile whose rings are being filled (set by begin_tile) ----
  // wave-uniform sources of the direct-to-LDS loads:
  // A slice: 32 regions of 1 KiB (8 rows x 128 B), kAReg per wave.
  // B stage: 16 regions of 1 KiB (2 rows x 512 B), kBReg per wave.
  int m0 = 0, n0 = 0;
  const char *ua = nullptr, *ub = nullptr;
  const int64_t a_region = (int64_t)K * 16;   // 8 rows of A
  const int64_t b_region = (int64_t)N * 4;    // 2 rows of B
  int ka_next = 0;  // slice (64 k) the next A issue fetches
  int kb_next = 0;  // stage (32 k) the next B issue fetches
  // K-stagger: a tile walks stages kfirst, kfirst+1, ..., wrapping at KT.
  // kfirst is even so that A slices (two stages) stay aligned.
  auto first_stage = [&](int tile_m, int tile_n) {
    return (int)(((unsigned)(tile_m * AFIR_MM_KSTAGGER_M + tile_n * AFIR_MM_KSTAGGER_N) * 2u) % (unsigned)KW);
  };
  auto begin_tile = [&](int p) {
    int tile_m, tile_n;
    map_tile_dma(p, tiles_m, tiles_n, tile_m, tile_n);
    m0 = tile_m * kBM;
    n0 = tile_n * kBN;
    if (kPrefetch > 0 && !feeder) return;   // those waves keep a cursor of their own in ua / ub
    const int kfirst = first_stage(tile_m, tile_n);
    ua = reinterpret_cast<const char *>(A) +
         ((int64_t)(m0 + wave * (kAReg * 8)) * K + (int64_t)kfirst * kBK) * 2;
    const uint16_t *b_of_batch = B;
    if constexpr (Batched) b_of_batch += (int64_t)(tile_m / tiles_m_batch) * b_batch_stride;
    ub = reinterpret_cast<const char *>(b_of_batch) +
         ((int64_t)(wave * (kBReg * 2) + kfirst * kBK) * N + n0) * 2;
    ka_next = kfirst >> 1;
    kb_next = kfirst;
  };
  // ---- prefetch (kPrefetch > 0; the waves that feed nothing) ----
  // A cursor walks the sequence of (tile, stage) that the multiply walks, kPrefetch stages ahead
  // of it and across tile boundaries, a pair of stages per pair of steps: the A slice's 256
  // lines (one per row) at an even step, the two B stages' 256 lines (four per row) at an odd
  // one, a quarter of each per prefetching wave.  The loads ask for one dword per line and
  // nothing waits for them; what they leave behind is the line in the XCD's L2.  The cursor
  // lives in the registers of the feed cursor, which these waves do not use: ua / ub the
  // sources, ka_next the slice, pf_left the stages left in the cursor's tile.
  int pf_tile = 0, pf_left = 0;
  auto pf_seek = [&](int p, int ahead) {   // cursor to tile p, `ahead` (even) stages into its walk
    int tile_m, tile_n;
    map_tile_dma(p, tiles_m, tiles_n, tile_m, tile_n);
    const int k = (first_stage(tile_m, tile_n) + ahead) % KW;
    const int pw = wave - kFeedWaves;
    ua = reinterpret_cast<const char *>(A) + ((int64_t)(tile_m * kBM + pw * 64) * K + (int64_t)k * kBK) * 2;
    const uint16_t *b_of_batch = B;
    if constexpr (Batched) b_of_batch += (int64_t)(tile_m / tiles_m_batch) * b_batch_stride;
    ub = reinterpret_cast<const char *>(b_of_batch) + ((int64_t)(k * kBK + pw * 16) * N + tile_n * kBN) * 2;
    ka_next = k >> 1;
    pf_tile = p;
    pf_left = KT - ahead;
  };
  auto pf_load = [&](const char *base, uint32_t lane_offset) {
    asm volatile("global_load_dword %0, %1, %2" : "+v"(a_lane[1]) : "v"(lane_offset), "s"(base) : "memory");
  };
  auto pf_advance = [&]() {   // on by a pair of stages; to the next tile of this workgroup at the end
    pf_left -= 2;
    if (pf_left > 0) {
      const bool wrap = ka_next + 1 == KW2;
      ka_next = wrap ? 0 : ka_next + 1;
      ua += wrap ? -(int64_t)(KW2 - 1) * 128 : (int64_t)128;
      ub += (wrap ? -(int64_t)(KW - 2) : (int64_t)2) * kBK * N * 2;
    } else if (pf_tile + (int)gridDim.x < tiles_m * tiles_n) {
      pf_seek(pf_tile + (int)gridDim.x, 0);
    }
  };
  // one region: lane l's 16 bytes go to lds_offset + 16 l
  auto dma = [&](const char *base, uint32_t lane_offset, uint32_t lds_offset) {
    Feed::source(base, lane_offset, A, lane);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(lds_offset), "v"(lane_offset), "s"(base)
                 : "memory");
  };
  auto issue_a_region = [&](int slot, auto q_tag) {
    constexpr int q = decltype(q_tag)::value;
    dma(ua + q * a_region, a_lane[q & 1],
        lds_base + (uint32_t)(slot * kSlotA + wave * (kAReg * 1024) + q * 1024));
  };
  auto advance_a = [&]() {
    ka_next = (ka_next + 1 == KW2) ? 0 : ka_next + 1;
    ua += (ka_next == 0) ? -(int64_t)(KW2 - 1) * 128 : (int64_t)128;
  };
  auto issue_b_region = [&](int slot, auto q_tag) {
    constexpr int q = decltype(q_tag)::value;
    dma(ub + q * b_region, b_lane[q & 1],
        lds_base + (uint32_t)(kRingB + slot * kSlotB + wave * (kBReg * 1024) + q * 1024));
  };
  auto advance_b = [&]() {
    kb_next = (kb_next + 1 == KW) ? 0 : kb_next + 1;
    ub += ((kb_next == 0) ? -(int64_t)(KW - 1) : (int64_t)1) * kBK * N * 2;
  };
  auto issue_a = [&](int slot) {
    static_for<0, kAReg>([&](auto q) { issue_a_region(slot, q); });
    advance_a();
  };
  // The fill of both rings at the start of a tile, oldest first: A(0) B(0) B(1) A(1) B(2) B(3)
  // A(2) (the launcher guarantees KT >= 8).  All of it but A(2) is issued *during the epilogue
  // of the previous tile*, one region behind each block of epilogue arithmetic: the rings are
  // free once every wave has left the K loop, the epilogue stages its rows in A slot 2, and so
  // the first stages of the next tile are in LDS (and the issue cost of 160 KiB of loads is paid
  // behind vector arithmetic) by the time the epilogue's last store is out.  The float32 output
  // form needs twice the staging room and keeps the whole fill after its epilogue.
  constexpr bool kEarlyFill = !F16IO;
  constexpr int kEarlyRegions = 2 * kAReg + 4 * kBReg;
  auto early_fill_item = [&](auto x_tag) {
    constexpr int X = decltype(x_tag)::value;
    constexpr int a0 = 0, b0 = kAReg, b1 = b0 + kBReg, a1 = b1 + kBReg, b2 = a1 + kAReg, b3 = b2 + kBReg;
    if constexpr (X < b0) issue_a_region(0, std::integral_constant<int, X - a0>{});
    else if constexpr (X < b1) issue_b_region(0, std::integral_constant<int, X - b0>{});
    else if constexpr (X < a1) issue_b_region(1, std::integral_constant<int, X - b1>{});
    else if constexpr (X < b2) issue_a_region(1, std::integral_constant<int, X - a1>{});
    else if constexpr (X < b3) issue_b_region(2, std::integral_constant<int, X - b2>{});
    else issue_b_region(3, std::integral_constant<int, X - b3>{});
    if constexpr (X == b0 - 1 || X == b2 - 1) advance_a();
    if constexpr (X == b1 - 1 || X == a1 - 1 || X == b3 - 1 || X == kEarlyRegions - 1) advance_b();
  };

  const int total_tiles = tiles_m * tiles_n;
  if ((int)blockIdx.x < total_tiles) {
    begin_tile(blockIdx.x);
    if (feeder) {
      static_for<0, kEarlyRegions>([&](auto x) { early_fill_item(x); });
      issue_a(2);
    } else if (kPrefetch > 0) {
      pf_seek(blockIdx.x, kPrefetch);
    }
  }
  for (int p = blockIdx.x; p < total_tiles; p += gridDim.x) {
    // the tile being computed (m0 / n0 move on to the next tile during the epilogue)
    const int out_m0 = m0, out_n0 = n0;
    const bool has_next_tile = p + (int)gridDim.x < total_tiles;

    f32x4 acc[kTM][kTN];
#pragma unroll
    for (int i = 0; i < kTM; ++i)
#pragma unroll
      for (int j = 0; j < kTN; ++j)
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[i][j][e] = 0.f;

    // LDS addresses of a stage held in A slot sa / B slot sbk; the stage is the first
    // (par 0) or second (par 1) half of its A slice
    auto a_address = [&](int sa, int par) {
      return lds_base + (uint32_t)(sa * kSlotA) + (a_rd ^ (uint32_t)(par * 64));
    };
    auto b_addresses = [&](int sbk, uint32_t (&ba)[kTN]) {
      const uint32_t bb = lds_base + (uint32_t)(sbk * kSlotB) + b_rd0;   // ring slots are 1 KiB aligned
#pragma unroll
      for (int j = 0; j < kTN; ++j) ba[j] = bb ^ (uint32_t)(j * 32);
    };

    // the rings were filled before the loop or during the previous epilogue.  At most the loads
    // younger than A(0), B(0) may be outstanding; stores of the previous epilogue that are still
    // on their way only make this wait stricter (loads complete in order among themselves, so
    // A(0) or B(0) outstanding means all the younger loads are too: more than the bound).
    if (feeder) wait_vmcnt<3 * kBReg + 2 * kAReg>();
    __builtin_amdgcn_s_barrier();
    // Operand registers: the A fragments of a stage in two halves (m tiles 0-3, 4-7), the B
    // fragments of a stage twice (the stage being multiplied and the next one).
    u32x4 a_lo[4], a_hi[4];
    u32x2 b_cur[kTN][2], b_nxt[kTN][2];
    {
      uint32_t ba[kTN];
      b_addresses(0, ba);
      issue_a_reads<0>(a_address(0, 0), a_lo);
      issue_b_reads(ba, b_cur);
      settle_wait();
      settle(a_lo);
      settle(b_cur);
    }
    if (!Feed::kOperandReads) {   // the registers the loop would have read into hold something
#pragma unroll
      for (int i = 0; i < 4; ++i) a_hi[i] = a_lo[i];
#pragma unroll
      for (int j = 0; j < kTN; ++j) {
        b_nxt[j][0] = b_cur[j][0];
        b_nxt[j][1] = b_cur[j][1];
      }
    }

    // One step of the pipeline for stage s (parity PAR within its A slice), the B
    // fragments of s in `bs`, those of s+1 going to `bn`:
    //   reads of A(s) m tiles 4-7 in flight | MFMAs of m tiles 0-3
    //   wait until stage s+1 has landed, barrier: everyone is done reading s
    //   reads of A(s+1) m tiles 0-3 and B(s+1) in flight, refill the freed slots
    //                                        | MFMAs of m tiles 4-7
    // Refill after stage s: B(s+4) into s's B slot, right after the barrier of step s; after
    // an odd s also the A slice (s+5)/2 into the slot of the slice just finished, behind the
    // first MFMAs of step s+1.  In the steady state both exist and the vmcnt is exact: the
    // loads younger than what stage s+1 needs are 2 B stages and 2 A slices at an even s
    // (B(s+2), B(s+3), and the slices issued in steps s-2 and s), 2 B stages and 1 A slice at
    // an odd s.  Otherwise drain.
    int sa = 0, sb = 0;  // ring slots of the stage being multiplied
    // (opaque: with known slots the compiler precomputes the operand addresses of the first two
    // steps once per kernel, spills them, and the reload waits for the whole ring fill)
    asm volatile("" : "+s"(sa), "+s"(sb));
    auto pin = [] { __builtin_amdgcn_sched_barrier(0); };
    // MFMA number X of a phase: n tile X / 4, m tile FIRST + X % 4
    auto mfma = [&](auto first_tag, auto x_tag, const u32x4 (&a)[4], const u32x2 (&b)[kTN][2]) {
      constexpr int FIRST = decltype(first_tag)::value, X = decltype(x_tag)::value;
      constexpr int j = AFIR_MM_MFMA_A_OUTER ? X % 4 : X / 4, i = AFIR_MM_MFMA_A_OUTER ? X / 4 : X % 4;
      const u32x4 bw = {b[j][0].x, b[j][0].y, b[j][1].x, b[j][1].y};
      if constexpr (F16IO)
        acc[FIRST + i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
            __builtin_bit_cast(f16x8, bw), __builtin_bit_cast(f16x8, a[i]), acc[FIRST + i][j], 0, 0, 0);
      else
        acc[FIRST + i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
            __builtin_bit_cast(bf16x8, bw), __builtin_bit_cast(bf16x8, a[i]), acc[FIRST + i][j], 0, 0, 0);
    };
    // The A refill waits for the step after the one that frees its slot, so that it goes out
    // behind the MFMAs of phase 1, which carries few operand reads: pend_a says whether the
    // previous step left one to issue, pend_sa into which slot (pend_b / pend_sb: the same for
    // the B stage when AFIR_MM_B_EARLY is 0).
    bool pend_a = false, pend_b = false;
    int pend_sa = 0, pend_sb = 0;
    // pend_tag: what is known at compile time about the refills the previous step left: 0 none
    // (the first step of a tile), 1 those of the steady state (a B stage; an A slice after an
    // odd stage), 2 whatever pend_a / pend_b say
    auto step = [&](auto par_tag, auto mode_tag, auto pend_tag, u32x2 (&bs)[kTN][2], u32x2 (&bn)[kTN][2],
                    bool has_next, bool refill_b, bool refill_a) {
      constexpr int PAR = decltype(par_tag)::value;
      constexpr bool STEADY = decltype(mode_tag)::value;
      constexpr int PEND = decltype(pend_tag)::value;
      constexpr int NM = 4 * kTN;   // MFMAs per phase
      const int sb_next = (sb + 1 == kBSlots) ? 0 : sb + 1;
      const int sa_next = PAR ? ((sa + 1 == kASlots) ? 0 : sa + 1) : sa;
      // ---- phase 1: m tiles 0-3.  One item behind each MFMA: the reads of m tiles 4-7 first
      // (they have the rest of the phase to come back), then the refills the previous step
      // left (its A slice, if any, before its B stage).
      {
        const uint32_t aa = a_address(sa, PAR);
        const bool do_a = Feed::kLoads && feeder && (PEND == 1 ? !PAR : PEND == 2 && pend_a);
        const bool do_b = !AFIR_MM_B_EARLY && Feed::kLoads && feeder && (PEND == 1 || (PEND == 2 && pend_b));
        pin();
        static_for<0, NM>([&](auto x) {
          constexpr int X = decltype(x)::value;
          mfma(std::integral_constant<int, 0>{}, x, a_lo, bs);
          pin();
          // MFMAs between two refill loads (every MFMA when a wave has twelve slots' worth to issue)
          constexpr int kStride = kAReg + (AFIR_MM_B_EARLY ? 0 : kBReg) > 6 ? 1 : AFIR_MM_DMA_STRIDE;
          constexpr int I = X >= 4 && (X - 4) % kStride == 0 ? (X - 4) / kStride : -1;
          if constexpr (X < 4) {
            if (Feed::kOperandReads) read_a<(4 + X) * 2048>(aa, a_hi[X]);
            pin();
          } else if constexpr (!PAR && I >= 0 && I < kAReg) {   // the step before an even stage was odd: A slice
            if (do_a) issue_a_region(pend_sa, std::integral_constant<int, I>{});
            pin();
          } else if constexpr (I >= kAReg && I < kAReg + kBReg) {
            if (do_b) issue_b_region(pend_sb, std::integral_constant<int, I - kAReg>{});
            pin();
          }
          if constexpr (kPrefetch > 0 && X == 6) {
            if (!feeder && pf_left > 0) {
              if constexpr (!PAR) pf_load(ua, a_lane[0]);
              else pf_load(ub, b_lane[0]);
            }
            pin();
          }
        });
        if (do_a) advance_a();
        if (do_b) advance_b();
        if (kPrefetch > 0 && PAR && !feeder && pf_left > 0) pf_advance();
      }
      pin();
      settle_wait();
      settle(a_hi);
      pin();
      // ---- phase 2: m tiles 4-7.  Behind the first MFMA: wait until stage s+1 has landed,
      // barrier (everyone is done reading s); then one operand read of stage s+1 behind each
      // of the next twelve MFMAs, in the order the next phase uses them.
      if (STEADY || has_next) {
        uint32_t ba[kTN];
        b_addresses(sb_next, ba);
        const uint32_t aa = a_address(sa_next, PAR ^ 1);
        static_for<0, NM>([&](auto x) {
          constexpr int X = decltype(x)::value;
          mfma(std::integral_constant<int, 4>{}, x, a_hi, bs);
          pin();
          if constexpr (X == 0) {
            if (feeder) {   // the other waves issued none of the loads a stage consists of
              if (STEADY)
                wait_vmcnt<AFIR_MM_B_EARLY ? (PAR ? 2 * kBReg + kAReg : 2 * kBReg + 2 * kAReg) : kSteadyVm>();
              else
                wait_vmcnt<0>();
            }
            __builtin_amdgcn_s_barrier();
            pin();
          }
          if constexpr (X < 12) {
            constexpr int R = X;   // B tile 0, A tiles 0-3, B tiles 1-3
            if (Feed::kOperandReads) {
              if constexpr (R < 2) read_b<R * 4 * 512>(ba[0], bn[0][R]);
              else if constexpr (R < 6) read_a<(R - 2) * 2048>(aa, a_lo[R - 2]);
              else read_b<((R - 6) % 2) * 4 * 512>(ba[1 + (R - 6) / 2], bn[1 + (R - 6) / 2][(R - 6) % 2]);
            }
            pin();
          }
          if constexpr (AFIR_MM_B_EARLY && X >= 1 && X < 1 + kBReg) {
            // everyone is past the barrier: stage s is read, its B slot takes stage s + 4
            if (Feed::kLoads && feeder && (STEADY || refill_b))
              issue_b_region(sb, std::integral_constant<int, X - 1>{});
            pin();
          }
        });
        if (AFIR_MM_B_EARLY && Feed::kLoads && feeder && (STEADY || refill_b)) advance_b();
        pend_b = !AFIR_MM_B_EARLY && (STEADY || refill_b);
        pend_a = PAR && (STEADY || refill_a);
        pend_sa = sa;
        pend_sb = sb;
        pin();
        settle_wait();
        settle(a_lo);
        settle(bn);
      } else {
        static_for<0, NM>([&](auto x) { mfma(std::integral_constant<int, 4>{}, x, a_hi, bs); });
        pend_a = pend_b = false;
      }
      pin();
      sa = sa_next;
      sb = sb_next;
    };

    using Pend0 = std::integral_constant<int, 0>;
    using Pend1 = std::integral_constant<int, 1>;
    using Pend2 = std::integral_constant<int, 2>;
    // KT >= 8 (the launcher checks): the first two stages are steady ones
    step(Par0{}, Steady{}, Pend0{}, b_cur, b_nxt, true, true, true);
    step(Par1{}, Steady{}, Pend1{}, b_nxt, b_cur, true, true, true);
    int s = 2;
    for (; s + 6 < KT; s += 2) {  // both refills exist: B(s+4), B(s+5), A((s+6)/2)
      step(Par0{}, Steady{}, Pend1{}, b_cur, b_nxt, true, true, true);
      step(Par1{}, Steady{}, Pend1{}, b_nxt, b_cur, true, true, true);
    }
    for (; s < KT; s += 2) {
      step(Par0{}, Drain{}, Pend2{}, b_cur, b_nxt, true, s + 4 < KT, false);
      step(Par1{}, Drain{}, Pend2{}, b_nxt, b_cur, s + 2 < KT, s + 5 < KT, s + 6 < KT);
    }

    // Epilogue.  Of each 16 x 16 block a lane holds m = lane%16 and the four
    // consecutive n = 4*(lane/16) + e, i.e. 8 bytes (bf16) or 16 bytes (float32)
    // of an output row: written straight to memory that is a fraction of a line
    // per row per instruction, and the partial lines of the bf16 form cost three
    // times the write traffic.  So each wave stages 32 rows of its tile (two m
    // tiles; 64 n = one or two 128-byte lines per row) in LDS and stores them as
    // full lines, eight or four rows per instruction.  The rings are free once
    // every wave has left the K loop; a wave's 4 or 8 KiB staging area is
    // private, and the LDS unit keeps a wave's accesses in order, so no further
    // barrier is needed until the staging room is refilled.  The 16-byte
    // chunk column is XOR-ed with a function of the row: conflict-free for the
    // 8- or 16-byte writes and for the 16-byte row reads.
    __builtin_amdgcn_s_barrier();
    if (has_next_tile) begin_tile(p + (int)gridDim.x);
    {
      constexpr int kOutBytes = F16IO ? 4 : 2;
      constexpr int CH = kTN * 16 * kOutBytes / 16;   // 16-byte chunks per staged row: 8 or 16
      constexpr int kRowBytes = CH * 16;       // 128 or 256
      constexpr int kRowsPerPass = 64 / CH;    // rows one store instruction covers
      // The lane number again, opaque to the compiler: everything per lane that the epilogue
      // needs (staging addresses, bias columns, output rows) is then computed here, once per
      // tile, instead of once per kernel.  Hoisted out of the tile loop those values do not fit
      // the register file beside the K loop, and a reload from scratch memory makes the compiler
      // wait for *every* outstanding memory operation - each store of the epilogue and the fill of
      // the next tile - before it goes on.
      int lane_e;
      asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(lane_e));
      const int li = lane_e & 15, g = lane_e >> 4;
      // bf16: A slot 2, which the early fill of the next tile leaves alone
      unsigned char *const stage = smem + (kEarlyFill ? 2 * kSlotA : 0) + wave * (32 * kRowBytes);
      const int rr = lane_e / CH, cc = lane_e % CH;
      // two 128-byte rows share a swizzle value (they span the same banks as
      // one 256-byte row)
      auto swz = [](int r) { return CH == 8 ? ((r >> 1) & 7) : (r & (CH - 1)); };
      typedef typename std::conditional<F16IO, f32x4, u32x2>::type BiasRaw;
      BiasRaw braw[kTN];
#pragma unroll
      for (int j = 0; j < kTN; ++j) {
        const int n = out_n0 + (wn * kTN + j) * 16 + 4 * g;
        // no bias: -0, the identity of the add
        if constexpr (F16IO)
          braw[j] = bias_v ? *reinterpret_cast<const f32x4 *>(static_cast<const float *>(bias_v) + n)
                           : f32x4{-0.f, -0.f, -0.f, -0.f};
        else
          braw[j] = bias_v ? *reinterpret_cast<const u32x2 *>(static_cast<const uint16_t *>(bias_v) + n)
                           : u32x2{0x80008000u, 0x80008000u};
      }
      // the activation is a launch argument: one copy of the passes per kind, chosen by a
      // wave-uniform branch, so that no value pays a select
      auto passes = [&](auto relu_tag) {
        constexpr bool RELU = decltype(relu_tag)::value;
        static_for<0, kTM / 2>([&](auto ip_tag) {
          constexpr int ip = decltype(ip_tag)::value;
          static_for<0, 2 * kTN>([&](auto hj_tag) {
            constexpr int half = decltype(hj_tag)::value / kTN, j = decltype(hj_tag)::value % kTN;
            const int lm = half * 16 + li;   // row within the 32 staged rows
            {
              float b0, b1, b2, b3;
              if constexpr (F16IO) {
                b0 = braw[j][0]; b1 = braw[j][1]; b2 = braw[j][2]; b3 = braw[j][3];
              } else {
                b0 = bf16_lo(braw[j].x); b1 = bf16_hi(braw[j].x);
                b2 = bf16_lo(braw[j].y); b3 = bf16_hi(braw[j].y);
              }
              // one region of the next tile's fill behind each block of arithmetic
              if constexpr (kEarlyFill && (ip * 2 + half) * kTN + j < kEarlyRegions) {
                if (has_next_tile && feeder)
                  early_fill_item(std::integral_constant<int, (ip * 2 + half) * kTN + j>{});
              }
              const f32x4 &c = acc[ip * 2 + half][j];
              float v0 = c[0] + b0;
              float v1 = c[1] + b1;
              float v2 = c[2] + b2;
              float v3 = c[3] + b3;
              v0 = fmaxf(v0, RELU ? 0.f : v0 * alpha);
              v1 = fmaxf(v1, RELU ? 0.f : v1 * alpha);
              v2 = fmaxf(v2, RELU ? 0.f : v2 * alpha);
              v3 = fmaxf(v3, RELU ? 0.f : v3 * alpha);
              if constexpr (F16IO) {
                const f32x4 w = {v0, v1, v2, v3};
                const int chunk = (j * 4 + g) ^ swz(lm);
                *reinterpret_cast<f32x4 *>(stage + lm * kRowBytes + chunk * 16) = w;
              } else {
                u32x2 w;
                w.x = pack_bf16_hw(v0, v1);
                w.y = pack_bf16_hw(v2, v3);
                const int chunk = (j * 2 + (g >> 1)) ^ swz(lm);
                *reinterpret_cast<u32x2 *>(stage + lm * kRowBytes + chunk * 16 + (g & 1) * 8) = w;
              }
            }
          });
#pragma unroll
          for (int tq = 0; tq < 32 / kRowsPerPass; ++tq) {
            const int r = rr + kRowsPerPass * tq;
            const u32x4 line =
                *reinterpret_cast<const u32x4 *>(stage + r * kRowBytes + ((cc ^ swz(r)) * 16));
            const int m = out_m0 + (wm * kTM + ip * 2) * 16 + r;
            unsigned char *const row = static_cast<unsigned char *>(out_v) +
                                       ((int64_t)m * N + out_n0 + wn * (kTN * 16)) * kOutBytes;
#if AFIR_MM_NT_STORE
            __builtin_nontemporal_store(line, reinterpret_cast<u32x4 *>(row + cc * 16));
#else
            *reinterpret_cast<u32x4 *>(row + cc * 16) = line;
#endif
          }
        });
      };
      if (relu) passes(std::true_type{});
      else passes(std::false_type{});
    }
    // every wave must be done with its staging rows before the rest of the next fill lands there
    __builtin_amdgcn_s_barrier();
    if (has_next_tile && feeder) {
      if constexpr (!kEarlyFill) static_for<0, kEarlyRegions>([&](auto x) { early_fill_item(x); });
      issue_a(2);
    }
  }
  if (kPrefetch > 0) {   // the register of the prefetch loads stays reserved until they are all back
    wait_vmcnt<0>();
    asm volatile("" ::"v"(a_lane[1]));
  }
}

inline bool supported(int64_t m, int64_t k, int64_t n) {
  return m % kBM == 0 && n % kBN == 0 && k % 64 == 0 && k >= 8 * kBK;
}

#ifndef AFIR_MM_GRID
#define AFIR_MM_GRID device_cus()
#endif

// batch > 1 (with Batched): `m` is the extent of one product; A and out hold `batch` of them one
// after the other, B likewise (k * n elements apart)
template <bool F16IO, typename Feed, bool Batched = false>
LaunchStatus launch(const char *name, const uint16_t *a, const uint16_t *b, const void *bias, void *out, int m,
                    int k, int n, float alpha, bool relu, uint32_t block_dim, hipStream_t stream, int batch = 1) {
  auto kernel = matmul_bias_leakyrelu_dma<F16IO, Feed, Batched>;
  static hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                               hipFuncAttributeMaxDynamicSharedMemorySize,
                                               kLdsBytes);
  if (attr != hipSuccess) return LaunchStatus{2u, hipGetErrorString(attr)};
  if (!Batched && batch != 1) return LaunchStatus{1u, "matmul: this instance takes one product"};
  const int tiles_m_batch = m / kBM, tiles_m = tiles_m_batch * batch, tiles_n = n / kBN;
  // One workgroup fills a CU's LDS, so the grid is persistent: one workgroup
  // per CU, each walking its share of the tiles.
  int64_t blocks = (int64_t)tiles_m * tiles_n;
  if (blocks > AFIR_MM_GRID) blocks = AFIR_MM_GRID;
  if (block_dim) blocks = block_dim;
  AFIR_LAUNCH(name, kernel, dim3((unsigned)blocks), dim3(kWaves * 64), kLdsBytes, stream, a, b,
              bias, out, m * batch, k, n, alpha, relu ? 1 : 0, tiles_m, tiles_n, tiles_m_batch, (int64_t)k * n);
  return after_launch();
}

}  // namespace dma

}  // namespace afir
