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
#include "matmul_dma_kernel.h"

namespace afir {

bool matmul_dma_supported(int64_t m, int64_t k, int64_t n) { return dma::supported(m, k, n); }

LaunchStatus launch_matmul_dma(const uint16_t *a, const uint16_t *b, const uint16_t *bias,
                               uint16_t *out, int m, int k, int n, float alpha, bool relu,
                               uint32_t block_dim, hipStream_t stream) {
  return dma::launch<false, dma::FullFeed>("matmul_bias_leakyrelu_dma", a, b, bias, out, m, k, n, alpha, relu,
                                           block_dim, stream);
}

LaunchStatus launch_matmul_dma_f16(const uint16_t *a, const uint16_t *b, const float *bias,
                                   float *out, int m, int k, int n, float alpha, bool relu,
                                   uint32_t block_dim, hipStream_t stream) {
  return dma::launch<true, dma::FullFeed>("matmul_bias_leakyrelu_dma_f16", a, b, bias, out, m, k, n, alpha, relu,
                                          block_dim, stream);
}

LaunchStatus launch_matmul_dma_batched(const uint16_t *a, const uint16_t *b, const void *bias, void *out, bool f16io,
                                       int batch, int m, int k, int n, float alpha, bool relu, hipStream_t stream) {
  if (f16io)
    return dma::launch<true, dma::FullFeed, true>("matmul_bias_leakyrelu_dma_f16_batched", a, b, bias, out, m, k, n, alpha,
                                                  relu, 0, stream, batch);
  return dma::launch<false, dma::FullFeed, true>("matmul_bias_leakyrelu_dma_batched", a, b, bias, out, m, k, n, alpha, relu,
                                                 0, stream, batch);
}

}  // namespace afir
