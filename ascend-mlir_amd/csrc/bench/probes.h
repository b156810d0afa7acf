/*
 * Measurement aids of the benchmark (libafir_bench_probes.so).  Not part of the
 * drop-in boundary: nothing in the kernel or runtime libraries uses them, and
 * only bench.py loads this library.  They answer "what does this chip sustain
 * on the access pattern / instruction mix of a workload when nothing else
 * happens", so that a kernel's figure can be read against a measured ceiling
 * next to the published peak.  No counterpart in the reference.
 *
 * All pointers are device pointers; `stream` is a hipStream_t (NULL = default);
 * launches are asynchronous and the caller times them with events on `stream`.
 * Return 0 on success, 1 for bad arguments, 2 when HIP reports a launch error.
 */
#ifndef AFIR_BENCH_PROBES_H
#define AFIR_BENCH_PROBES_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Issues v_mfma_f32_16x16x32_bf16 (the matmul kernel's instruction) from registers on every CU (8 waves per
 * workgroup, two workgroups per CU) and nothing else.  `operands` = 65536 bytes
 * of bf16 (the VALUES matter: the sustained clock under the board power limit
 * depends on how much the operands toggle), `sink` = 1 MiB that receives one
 * float per lane.  *flops = floating-point operations of the launch. */
#define AFIR_BENCH_MFMA_OPERAND_BYTES 65536u
#define AFIR_BENCH_MFMA_SINK_BYTES 1048576u
uint32_t afir_bench_mfma_rate(void *stream, const void *operands, void *sink, uint32_t iters,
                              uint64_t *flops);

/* The direct-to-LDS matmul kernel (csrc/kernels/matmul_dma_kernel.h, instantiated here
 * with the feed policies of matmul_feed_probes.h) with parts of its K loop removed, so that a
 * matmul's distance from the register-only MFMA rate can be split into its
 * causes on the workload's own operands:
 *   what = 1  no global -> LDS feed after the prologue: the MFMAs, their LDS
 *             operand reads, waits and barriers remain (operands stay those of
 *             the first K steps);
 *   what = 2  no LDS operand reads either: MFMAs on the registers the first
 *             reads filled, waits and barriers remain;
 *   what = 3  the whole kernel, but every global -> LDS load reads the same
 *             1 KiB: the loads are issued and write LDS as always, without the
 *             L2 / fabric / HBM traffic and latency behind them;
 *   what = 4  the whole kernel with real addresses, but the walk over K wraps
 *             after 256 k, so that an XCD's operand panels stay in its L2:
 *             every load is an L2 hit (1 -> 3 -> 4 -> the kernel: issue cost,
 *             cost of L2 hits, cost of L2 misses).
 * Same arguments as the kernel's launcher (bf16 A [m,k], B [k,n], bias [n], out
 * [m,n]; m, n multiples of 256, k of 64); the output is meaningless. */
uint32_t afir_bench_matmul_ablated(void *stream, const void *a, const void *b, const void *bias,
                                   void *out, int m, int k, int n, int what);

/* Grid-strided copy, 128-bit non-temporal loads and stores, four in flight per
 * lane: the fastest of the load / store policy pairs for a stream that comes
 * from HBM and writes as much as it reads (5.90 TB/s; ordinary loads 5.76,
 * ordinary stores 5.5-5.7).  bytes must be a multiple of 16384. */
uint32_t afir_bench_copy(void *stream, const void *src, void *dst, size_t bytes);

/* Write-only stream: every lane stores a value of its own (128-bit non-temporal
 * stores, grid-strided).  bytes must be a multiple of 16384. */
uint32_t afir_bench_fill(void *stream, void *dst, size_t bytes, uint32_t seed);

/* The copy with the chip's reads and writes separated in time, the way the
 * one-shot gather and transpose kernels do it: every lane of the launch is
 * resident at once (2048 lanes per CU, eight 16-byte chunks each, so at most
 * 64 MiB on 256 CUs), requests all its chunks, and holds its stores back until
 * the real-time counter says the chip's reads have been served (300 ns + bytes
 * at 6.7 TB/s after the workgroup's start).  bytes must be a multiple of 32768. */
uint32_t afir_bench_copy_phased(void *stream, const void *src, void *dst, size_t bytes);

/* Read-only stream: every lane sums what it loads (128-bit non-temporal loads)
 * and one float per workgroup goes to `sink` (>= 8192 floats). */
uint32_t afir_bench_read(void *stream, const void *src, void *sink, size_t bytes);

/* The address pattern of a batched transpose walked in 64 x 64 tiles of 2-byte
 * elements, without the transposition: a workgroup loads the 64 runs of 128
 * bytes of tile (b, tm, tn) of x [nb, m, n] (ordinary loads) and stores 64 runs
 * of 128 bytes (non-temporal) where the tile's transpose lies in out [nb, n, m],
 * registers only (the values
 * written are those loaded, in load order).  m, n multiples of 64. */
uint32_t afir_bench_tilecopy64(void *stream, const void *x, void *out, int nb, int m, int n);

#ifdef __cplusplus
}
#endif
#endif
