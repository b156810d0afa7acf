// Row gather fused with scale and shift, f16:
//   out[r,:] = f16(table[idx[r],:] * scale + shift)
// (the fused gather region of --fuse-gather-elementwise,
// lib/Conversion/FuseGatherElementwise/FuseGatherElementwisePass.cpp:61-303, in
// the embedding flavour lib/Conversion/MarkStructuredOps/MarkStructuredOpsPass.cpp:141-145;
// golden style examples/gather-elementwise-fusion/gen_data.py:62-67: f32
// arithmetic, one round-to-nearest-even to f16).
//
// HBM-bound: each gathered row is read once and written once.  Four kernels, picked by the
// launcher: rows of 32 * 2^k halves, up to twice what fits the chip at once, take the kernel that
// separates the chip's reads from its writes in time (gather_scale_shift_f16_phased), larger
// launches of such rows the grouped kernel, other 16-byte aligned rows the kernel in which a lane owns one
// column chunk for the whole launch (gather_scale_shift_f16_vec), anything else the element
// kernel.  The product of two f16 values is exact in f32, so the fused multiply-add they share
// rounds exactly like the unfused golden.
#include "kernels.h"

namespace afir {

namespace {

#ifndef AFIR_GATHER_RIF
#define AFIR_GATHER_RIF 1
#endif
#ifndef AFIR_GATHER_PASSES
#define AFIR_GATHER_PASSES 4
#endif
constexpr int kThreads = 256;
constexpr int kRowsInFlight = AFIR_GATHER_RIF;
constexpr int kPassesPerBlock = AFIR_GATHER_PASSES;

// t * s + h on eight halves, parameters kept as f16 pairs.  The product of two f16 values is
// exact in float32 (11 x 11 significant bits), so the fused multiply-add rounds exactly where
// the float32 multiply followed by the float32 add of the golden rounds: once, at the add.
// Written this way each pair costs two v_fma_mix_f32 (f16 operands read in place) and one
// v_cvt_pk_f16_f32 instead of six conversions, two multiplies, two adds and a pack; with the
// row loads of 32768 rows in flight that arithmetic was 10 % of the kernel's time.
__device__ __forceinline__ u32x4 scale_shift_packed(u32x4 t, u32x4 s, u32x4 h) {
  typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
  u32x4 r;
#pragma unroll
  for (int d = 0; d < 4; ++d) {
    // (copies first: __builtin_bit_cast applied to a vector element reads element 0 with this compiler)
    const uint32_t tw = t[d], sw = s[d], hw = h[d];
    const half2_t tv = __builtin_bit_cast(half2_t, tw), sv = __builtin_bit_cast(half2_t, sw),
                  hv = __builtin_bit_cast(half2_t, hw);
    // (the empty asm keeps the float32 results as values of their own: left alone, the compiler
    // folds the conversion into the multiply-add in some contexts (v_fma_mixlo_f16), which rounds
    // once, to f16, where the golden rounds to float32 first)
    float lo = __builtin_fmaf((float)tv.x, (float)sv.x, (float)hv.x);
    float hi = __builtin_fmaf((float)tv.y, (float)sv.y, (float)hv.y);
    asm("" : "+v"(lo), "+v"(hi));
    half2_t o;
    o.x = (_Float16)lo;
    o.y = (_Float16)hi;
    r[d] = __builtin_bit_cast(uint32_t, o);
  }
  return r;
}

// dim % 8 == 0, 16-byte aligned buffers.  The workgroup is laid out as
// (lanes_per_row x rows_per_pass): lanes_per_row = min(256, dim/8 rounded up
// to a multiple of 64) so that a wave never straddles two rows.
__global__ __launch_bounds__(kThreads) void gather_scale_shift_f16_vec(
    const uint16_t *__restrict__ table, const int32_t *__restrict__ idx,
    const uint16_t *__restrict__ scale, const uint16_t *__restrict__ shift,
    uint16_t *__restrict__ out, int32_t *__restrict__ error_flag, uint32_t rows, int chunks,
    int64_t nidx, int lanes_per_row, int64_t rows_per_block) {
  const int rows_per_pass = kThreads / lanes_per_row;
  // a wave never straddles two rows, so the row slot is wave-uniform: say so,
  // and the index fetch becomes a scalar load
  const int slot = __builtin_amdgcn_readfirstlane(threadIdx.x / lanes_per_row);
  const int lane_col = threadIdx.x - slot * lanes_per_row;
  const int64_t dim = (int64_t)chunks * 8;
  const u32x4 nan_row = {0x7e007e00u, 0x7e007e00u, 0x7e007e00u, 0x7e007e00u};

  for (int64_t blk = blockIdx.x; blk * rows_per_block < nidx; blk += gridDim.x) {
    const int64_t r_begin = blk * rows_per_block;
    const int64_t r_end = (r_begin + rows_per_block < nidx) ? r_begin + rows_per_block : nidx;
    for (int col = lane_col; col < chunks; col += lanes_per_row) {
      u32x4 sraw = *reinterpret_cast<const u32x4 *>(scale + (int64_t)col * 8);
      u32x4 hraw = *reinterpret_cast<const u32x4 *>(shift + (int64_t)col * 8);
      for (int64_t r = r_begin + slot; r < r_end; r += (int64_t)rows_per_pass * kRowsInFlight) {
        // Branch-free fetch: rows past the end re-read the last row, indices
        // outside the table read row 0; both are discarded below.  All index
        // loads are issued first, then all row loads, so kRowsInFlight rows
        // are in flight per lane.
        uint32_t src[kRowsInFlight];
        bool good[kRowsInFlight];
        u32x4 v[kRowsInFlight];
#pragma unroll
        for (int u = 0; u < kRowsInFlight; ++u) {
          const int64_t rr = r + (int64_t)u * rows_per_pass;
          src[u] = (uint32_t)idx[rr < r_end ? rr : r_end - 1];
        }
#pragma unroll
        for (int u = 0; u < kRowsInFlight; ++u) {
          good[u] = src[u] < rows;
          const uint32_t safe = good[u] ? src[u] : 0u;
          v[u] = load_nt(reinterpret_cast<const u32x4 *>(table + (int64_t)safe * dim) + col);
        }
#pragma unroll
        for (int u = 0; u < kRowsInFlight; ++u) {
          const int64_t rr = r + (int64_t)u * rows_per_pass;
          if (rr < r_end) {
            u32x4 res = good[u] ? scale_shift_packed(v[u], sraw, hraw) : nan_row;
            store_nt(reinterpret_cast<u32x4 *>(out + rr * dim) + col, res);
            if (!good[u] && error_flag && col == 0) atomicOr(error_flag, 1);
          }
        }
      }
    }
  }
}

// Rows of exactly lanes * 4 chunks (lanes a power of two <= 256): a row is
// spread over `lanes` lanes, each taking four 16-byte chunks `lanes` chunks
// apart, so a wave-level load covers contiguous runs of whole rows and every
// lane has four loads in flight; 256 / lanes rows per workgroup pass.  The
// lane's four scale / shift chunks stay in registers.
constexpr int kGroups = 4;
// Consecutive passes a workgroup takes, all their row loads in flight together (1, 2 and 4
// measured 26.2 / 26.5 / 27.3 us on the 32768 x 1024 gather).
// Workgroups per CU the grid is capped at (further rows are walked grid-strided).  Few, long-lived
// workgroups (2 ... 16 per CU) with the next block's indices requested ahead measured 1-10 % slower
// than one block of rows per workgroup on the 32768 x 1024 gather.
#ifndef AFIR_GATHER_GROUPED_WG_PER_CU
#define AFIR_GATHER_GROUPED_WG_PER_CU 64
#endif
#ifndef AFIR_GATHER_NT_LOADS
#define AFIR_GATHER_NT_LOADS 0
#endif
#ifndef AFIR_GATHER_GROUPED_PASSES
#define AFIR_GATHER_GROUPED_PASSES 2
#endif
constexpr int kGroupedPasses = AFIR_GATHER_GROUPED_PASSES;
// lanes of a workgroup of the grouped kernel: with more row groups per workgroup the scale / shift
// vectors are fetched for more rows at once
#ifndef AFIR_GATHER_GROUPED_THREADS
#define AFIR_GATHER_GROUPED_THREADS 1024
#endif
constexpr int kGroupedThreads = AFIR_GATHER_GROUPED_THREADS;

__global__ __launch_bounds__(kGroupedThreads) void gather_scale_shift_f16_grouped(
    const uint16_t *__restrict__ table, const int32_t *__restrict__ idx,
    const uint16_t *__restrict__ scale, const uint16_t *__restrict__ shift,
    uint16_t *__restrict__ out, int32_t *__restrict__ error_flag, uint32_t rows, int lanes_log2,
    int64_t nidx) {
  const int lanes = 1 << lanes_log2;
  const int rows_per_pass = kGroupedThreads >> lanes_log2;
  const int local_row = threadIdx.x >> lanes_log2;
  const int col0 = threadIdx.x & (lanes - 1);
  const int64_t dim = (int64_t)lanes * kGroups * 8;
  const u32x4 nan_row = {0x7e007e00u, 0x7e007e00u, 0x7e007e00u, 0x7e007e00u};
  // scale and shift: every row group of the workgroup needs the same lanes * kGroups chunks of
  // each.  Loaded by the lanes of each row group separately that is 128 bytes per lane, twice
  // what a lane gathers per pass; instead the workgroup fetches the two vectors once (one chunk
  // of each per lane and round), parks them in LDS and every lane picks its chunks up from
  // there.  The fetch goes out behind the first block's row loads, so it costs no latency.
  extern __shared__ u32x4 params[];            // scale chunks, then shift chunks
  const int nchunks = lanes * kGroups;          // chunks per row
  u32x4 sraw[kGroups], hraw[kGroups];
  bool staged = false;
  const int64_t rows_per_block = (int64_t)rows_per_pass * kGroupedPasses;
  for (int64_t r0 = (int64_t)blockIdx.x * rows_per_block; r0 < nidx; r0 += (int64_t)gridDim.x * rows_per_block) {
    // all indices of the block's passes, then all their row loads, then the stores: rows past
    // the end re-read the last row and indices outside the table read row 0, both dropped below
    uint32_t src[kGroupedPasses];
    bool good[kGroupedPasses];
    u32x4 v[kGroupedPasses][kGroups];
#pragma unroll
    for (int p = 0; p < kGroupedPasses; ++p) {
      const int64_t r = r0 + (int64_t)p * rows_per_pass + local_row;
      src[p] = (uint32_t)idx[r < nidx ? r : nidx - 1];
    }
#pragma unroll
    for (int p = 0; p < kGroupedPasses; ++p) {
      good[p] = src[p] < rows;
      const u32x4 *row = reinterpret_cast<const u32x4 *>(table + (int64_t)(good[p] ? src[p] : 0u) * dim);
#pragma unroll
      for (int u = 0; u < kGroups; ++u)
        v[p][u] = AFIR_GATHER_NT_LOADS ? __builtin_nontemporal_load(row + col0 + u * lanes) : row[col0 + u * lanes];
    }
    if (!staged) {   // (the trip count is the same for every lane of the workgroup)
      for (int c = threadIdx.x; c < nchunks; c += kGroupedThreads) {
        params[c] = *reinterpret_cast<const u32x4 *>(scale + (int64_t)c * 8);
        params[nchunks + c] = *reinterpret_cast<const u32x4 *>(shift + (int64_t)c * 8);
      }
      __syncthreads();
#pragma unroll
      for (int u = 0; u < kGroups; ++u) {
        sraw[u] = params[col0 + u * lanes];
        hraw[u] = params[nchunks + col0 + u * lanes];
      }
      staged = true;
    }
#pragma unroll
    for (int p = 0; p < kGroupedPasses; ++p) {
      const int64_t r = r0 + (int64_t)p * rows_per_pass + local_row;
      if (r >= nidx) continue;
      u32x4 *dst = reinterpret_cast<u32x4 *>(out + r * dim);
#pragma unroll
      for (int u = 0; u < kGroups; ++u)
        store_nt(dst + col0 + u * lanes, good[p] ? scale_shift_packed(v[p][u], sraw[u], hraw[u]) : nan_row);
      if (!good[p] && error_flag && col0 == 0) atomicOr(error_flag, 1);
    }
  }
}

// The same row layout for gathers that fit the chip in one go (every lane of every workgroup
// resident at once: 2048 lanes per CU at 64 registers, eight 16-byte chunks per lane), with the
// reads and the writes of the whole chip separated in time.  HBM serves a pure read stream and a
// pure write stream faster than their mixture (64 MiB copied: 22.7 us mixed; 10.7 + 11.2 us as a
// read kernel followed by a write kernel), so every lane requests all its chunks at once and
// holds its stores back until `hold_ticks` of the real-time counter have passed since its
// workgroup started: by then the reads of all workgroups, which start within a microsecond or
// two of each other, have been served.  The wait is bounded and only shapes the timing: the
// stores are the same whenever they leave.  Measured on the 32768 x 1024 gather: 23.9 -> 21.6 us;
// on 24576 rows 20.5 -> 16.4, 8192 rows 8.6 -> 6.4.  The hold that measured best is the time the
// gathered bytes take at AFIR_GATHER_PHASE_GBS plus AFIR_GATHER_PHASE_BASE_NS, for 8192 to 32768
// rows alike (a third of a microsecond either side costs 1 %).  The formula assumes rows that come
// from HBM; when they repeat and come out of the caches the reads end early, and a workgroup
// that sees its own loads back ahead of its place in the launch cuts its hold short
// (phase_hold_here in common.h): 32768 indices over 2048 distinct rows 17.0 us (23.2 without
// the cut, 16.0 on the kernel without a hold).
#ifndef AFIR_GATHER_PHASED
#define AFIR_GATHER_PHASED 1
#endif
// a workgroup whose own loads came back so early that its place in the launch predicts the end of
// the chip's reads before this percentage of the formula's hold waits only until then
// (phase_hold_here; 100: the shorter of the two, 0: always the formula)
#ifndef AFIR_PHASE_ESTIMATE
#define AFIR_PHASE_ESTIMATE 100
#endif
#ifndef AFIR_GATHER_PHASED_THREADS
#define AFIR_GATHER_PHASED_THREADS 256
#endif
#ifndef AFIR_GATHER_PHASE_GBS
#define AFIR_GATHER_PHASE_GBS 6500
#endif
#ifndef AFIR_GATHER_PHASE_BASE_NS
#define AFIR_GATHER_PHASE_BASE_NS 300
#endif
// Workgroups of kPhasedThreads lanes where eight of them fit a compute unit beside their scale /
// shift chunks in LDS; rows of 8192 halves park 32 KiB per workgroup, and then four workgroups of
// kPhasedWideThreads lanes keep the same 2048 lanes per CU resident (8192 x 8192 rows gathered:
// 44.8 us against 49.0 on the grouped kernel; 1024-half rows are 1.5 % slower this way).
constexpr int kPhasedThreads = AFIR_GATHER_PHASED_THREADS;
constexpr int kPhasedWideThreads = 512;
constexpr int kPhasedPasses = 2;
constexpr int kPhasedLanesPerCU = 2048;

template <int kWg>
__global__ __launch_bounds__(kWg, kPhasedLanesPerCU / kWg) void gather_scale_shift_f16_phased(
    const uint16_t *__restrict__ table, const int32_t *__restrict__ idx,
    const uint16_t *__restrict__ scale, const uint16_t *__restrict__ shift,
    uint16_t *__restrict__ out, int32_t *__restrict__ error_flag, uint32_t rows, int lanes_log2,
    int hold_ticks) {
  const long long t_start = wall_clock64();
  const int lanes = 1 << lanes_log2;
  const int rows_per_pass = kWg >> lanes_log2;
  const int local_row = threadIdx.x >> lanes_log2;
  const int col0 = threadIdx.x & (lanes - 1);
  const int dim = lanes * kGroups * 8;
  const int nchunks = lanes * kGroups;          // chunks per row
  extern __shared__ u32x4 params[];            // scale chunks, then shift chunks
  const int64_t r0 = (int64_t)blockIdx.x * (rows_per_pass * kPhasedPasses);

  uint32_t src[kPhasedPasses];
  bool good[kPhasedPasses];
  u32x4 v[kPhasedPasses][kGroups];
#pragma unroll
  for (int p = 0; p < kPhasedPasses; ++p) {
    src[p] = (uint32_t)idx[r0 + p * rows_per_pass + local_row];
  }
#pragma unroll
  for (int p = 0; p < kPhasedPasses; ++p) {
    good[p] = src[p] < rows;
    const u32x4 *row = reinterpret_cast<const u32x4 *>(table + (int64_t)(good[p] ? src[p] : 0u) * dim) + col0;
#pragma unroll
    for (int u = 0; u < kGroups; ++u) v[p][u] = row[u * lanes];
  }
  for (int c = threadIdx.x; c < nchunks; c += kWg) {
    params[c] = *reinterpret_cast<const u32x4 *>(scale + (int64_t)c * 8);
    params[nchunks + c] = *reinterpret_cast<const u32x4 *>(shift + (int64_t)c * 8);
  }
  // (the asm makes the loads' results exist here, so the wait for them sits before the hold)
#pragma unroll
  for (int p = 0; p < kPhasedPasses; ++p)
#pragma unroll
    for (int u = 0; u < kGroups; ++u) asm volatile("" : "+v"(v[p][u]));
  __syncthreads();
#if AFIR_PHASE_ESTIMATE
  hold_ticks = phase_hold_here(hold_ticks, t_start, AFIR_PHASE_ESTIMATE * 0.01f);
#endif
  for (int spin = 0; spin < kPhaseSpinLimit && wall_clock64() - t_start < hold_ticks; ++spin)
    __builtin_amdgcn_s_sleep(1);

  // stores: a base per (pass, chunk group) that is the same for the whole workgroup (scalar
  // registers) plus one 32-bit offset per lane.  The lane's scale / shift chunks come from LDS at
  // their use: held in registers across the loads they would push the kernel past 64 registers.
  const u32x4 nan_row = {0x7e007e00u, 0x7e007e00u, 0x7e007e00u, 0x7e007e00u};
  char *block_out = reinterpret_cast<char *>(out) + r0 * dim * 2;
  const uint32_t lane_off = (uint32_t)(local_row * dim + col0 * 8) * 2u;
#pragma unroll
  for (int u = 0; u < kGroups; ++u) {
    const u32x4 sraw = params[col0 + u * lanes], hraw = params[nchunks + col0 + u * lanes];
#pragma unroll
    for (int p = 0; p < kPhasedPasses; ++p) {
      char *base = block_out + ((int64_t)p * rows_per_pass * dim + (int64_t)u * lanes * 8) * 2;
      const u32x4 res = good[p] ? scale_shift_packed(v[p][u], sraw, hraw) : nan_row;
      // (s_nop: the store reads its four data registers over the following cycles)
      asm volatile("global_store_dwordx4 %0, %1, %2 nt\n\ts_nop 1" ::"v"(lane_off), "v"(res), "s"(base) : "memory");
    }
  }
  const bool bad = !(good[0] && good[1]);
  if (bad && error_flag && col0 == 0) atomicOr(error_flag, 1);
}

// Any dim / alignment: one wave per row, 2-byte accesses.
__global__ __launch_bounds__(kThreads) void gather_scale_shift_f16_any(
    const uint16_t *__restrict__ table, const int32_t *__restrict__ idx,
    const uint16_t *__restrict__ scale, const uint16_t *__restrict__ shift,
    uint16_t *__restrict__ out, int32_t *__restrict__ error_flag, uint32_t rows, int64_t dim,
    int64_t nidx) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t wave = (int64_t)blockIdx.x * (kThreads / kWave) + (threadIdx.x >> 6);
  const int64_t nwaves = (int64_t)gridDim.x * (kThreads / kWave);
  for (int64_t r = wave; r < nidx; r += nwaves) {
    const uint32_t src = (uint32_t)idx[r];
    const bool good = src < rows;
    if (!good && error_flag && lane == 0) atomicOr(error_flag, 1);
    for (int64_t j = lane; j < dim; j += kWave) {
      uint16_t res = 0x7e00u;
      if (good) {
        float t = (float)__builtin_bit_cast(_Float16, table[(int64_t)src * dim + j]);
        float s = (float)__builtin_bit_cast(_Float16, scale[j]);
        float h = (float)__builtin_bit_cast(_Float16, shift[j]);
        res = __builtin_bit_cast(uint16_t, (_Float16)(t * s + h));
      }
      out[r * dim + j] = res;
    }
  }
}

}  // namespace

LaunchStatus launch_gather_scale_shift(const uint16_t *table, const int32_t *idx,
                                       const uint16_t *scale, const uint16_t *shift,
                                       uint16_t *out, int32_t *error_flag, int64_t rows,
                                       int64_t dim, int64_t nidx, uint32_t block_dim,
                                       hipStream_t stream) {
  if (rows < 0 || dim < 0 || nidx < 0) return invalid("gather_scale_shift: negative extent");
  if (nidx == 0 || dim == 0) return ok_status();
  if (!idx || !out || !scale || !shift) return invalid("gather_scale_shift: null tensor pointer");
  if (rows > 0 && !table) return invalid("gather_scale_shift: null table pointer");
  if (rows > 0x7fffffffLL) return invalid("gather_scale_shift: table rows exceed int32 index range");
  if (dim > 0x7fffffffLL || nidx > INT64_MAX / dim / 4 || (rows && rows > INT64_MAX / dim / 4))
    return invalid("gather_scale_shift: extent overflow");

  // (an empty table has no row to fall back on: the scalar kernel never reads it)
  const bool vec = rows > 0 && (dim % 8 == 0) && aligned16(table) && aligned16(scale) && aligned16(shift) &&
                   aligned16(out);
  const int64_t chunks64 = dim / 8;
  int lanes_log2 = 0;
  while (lanes_log2 < 8 && ((int64_t)kGroups << lanes_log2) < chunks64) ++lanes_log2;
  // Whole blocks of rows go to the phased kernel, which wants every lane of a launch resident at
  // once: a gather of up to twice that goes out as two launches (kPhaseMaxLaunches).  Rows left
  // over, and larger gathers: below.
  // blocks per launch: what is resident at once, asked of the runtime with the launch's LDS (scale
  // and shift, 16-byte chunks).  With fewer resident lanes than 2048 per CU (five workgroups of 256
  // lanes on rows of 8192 halves) such launches measured 4-11 % behind the grouped kernel.
  const size_t lds = (size_t)2 * (kGroups << lanes_log2) * 16;
  int phased_threads = 0;
  if (AFIR_GATHER_PHASED && vec && lanes_log2 <= 8) {
    static int threads_for[9] = {0, 0, 0, 0, 0, 0, 0, 0, 0};   // per row length, asked once (0: not yet, -1: none)
    if (threads_for[lanes_log2] == 0) {
      threads_for[lanes_log2] = -1;
      if ((1 << lanes_log2) <= kPhasedThreads &&
          resident_blocks_per_cu(gather_scale_shift_f16_phased<kPhasedThreads>, kPhasedThreads, lds) >= kPhasedLanesPerCU / kPhasedThreads)
        threads_for[lanes_log2] = kPhasedThreads;
      else if (kPhasedWideThreads > kPhasedThreads &&
               resident_blocks_per_cu(gather_scale_shift_f16_phased<kPhasedWideThreads>, kPhasedWideThreads, lds) >=
                   kPhasedLanesPerCU / kPhasedWideThreads)
        threads_for[lanes_log2] = kPhasedWideThreads;
    }
    if (threads_for[lanes_log2] > 0) phased_threads = threads_for[lanes_log2];
  }
  const int64_t phased_rows_per_block = phased_threads ? (int64_t)(phased_threads >> lanes_log2) * kPhasedPasses : 1;
  const int64_t phased_blocks = phased_threads ? nidx / phased_rows_per_block : 0;
  const int64_t capacity = phased_threads ? (int64_t)device_cus() * (kPhasedLanesPerCU / phased_threads) : 0;
  // (a launch whose last wave of workgroups leaves many compute units idle gains nothing: 640
  // workgroups of 512 lanes on 256 CUs measured 5 % behind the grouped kernel)
  const auto fills_the_chip = [&](int64_t blocks) {
    const int64_t cus = device_cus(), waves = (blocks + cus - 1) / cus;
    return blocks <= cus || blocks * 10 >= waves * cus * 9;
  };
  if (AFIR_GATHER_PHASED && vec && ((int64_t)kGroups << lanes_log2) == chunks64 && !block_dim && capacity > 0 &&
      phased_blocks > 0 && phased_blocks <= kPhaseMaxLaunches * capacity && phased_enabled() &&
      fills_the_chip((phased_blocks + (phased_blocks + capacity - 1) / capacity - 1) / ((phased_blocks + capacity - 1) / capacity))) {
    const int base_ns = env_int("AFIR_GATHER_PHASE_BASE_NS", AFIR_GATHER_PHASE_BASE_NS, 0, 100000);
    const int gbs = env_int("AFIR_GATHER_PHASE_GBS", AFIR_GATHER_PHASE_GBS, 100, 100000);
    const int64_t launches = (phased_blocks + capacity - 1) / capacity;
    const int64_t take = (phased_blocks + launches - 1) / launches;
    for (int64_t b0 = 0; b0 < phased_blocks; b0 += take) {
      const int64_t nblocks = phased_blocks - b0 < take ? phased_blocks - b0 : take;
      const int64_t row0 = b0 * phased_rows_per_block;
      const int hold_ticks = phase_hold_ticks(nblocks * phased_rows_per_block * dim * 2, base_ns, gbs);
      if (phased_threads == kPhasedThreads)
        AFIR_LAUNCH("gather_scale_shift_f16_phased", gather_scale_shift_f16_phased<kPhasedThreads>, dim3((unsigned)nblocks),
                    dim3(kPhasedThreads), lds, stream, table, idx + row0, scale, shift, out + row0 * dim, error_flag,
                    (uint32_t)rows, lanes_log2, hold_ticks);
      else
        AFIR_LAUNCH("gather_scale_shift_f16_phased", gather_scale_shift_f16_phased<kPhasedWideThreads>, dim3((unsigned)nblocks),
                    dim3(kPhasedWideThreads), lds, stream, table, idx + row0, scale, shift, out + row0 * dim, error_flag,
                    (uint32_t)rows, lanes_log2, hold_ticks);
    }
    const int64_t done = phased_blocks * phased_rows_per_block;
    if (done == nidx) return after_launch();
    idx += done;
    out += done * dim;
    nidx -= done;
  }
  if (vec && ((int64_t)kGroups << lanes_log2) == chunks64) {
    const int64_t rows_per_block = (int64_t)(kGroupedThreads >> lanes_log2) * kGroupedPasses;
    int64_t blocks = (nidx + rows_per_block - 1) / rows_per_block;
    if (blocks > (int64_t)device_cus() * AFIR_GATHER_GROUPED_WG_PER_CU) blocks = (int64_t)device_cus() * AFIR_GATHER_GROUPED_WG_PER_CU;
    if (block_dim) blocks = block_dim;
    AFIR_LAUNCH("gather_scale_shift_f16_grouped", gather_scale_shift_f16_grouped, dim3((unsigned)blocks), dim3(kGroupedThreads), lds,
                       stream, table, idx, scale, shift, out, error_flag, (uint32_t)rows, lanes_log2,
                       nidx);
  } else if (vec) {
    const int chunks = (int)(dim / 8);
    int lanes_per_row = ((chunks + kWave - 1) / kWave) * kWave;
    if (lanes_per_row > kThreads) lanes_per_row = kThreads;
    if (lanes_per_row == 192) lanes_per_row = 256;  // must divide the workgroup
    const int rows_per_pass = kThreads / lanes_per_row;
    // rows handled by one workgroup before it moves on: enough to amortise the
    // scale/shift registers, small enough to spread over all CUs
    int64_t rows_per_block = (int64_t)rows_per_pass * kRowsInFlight * kPassesPerBlock;
    int64_t blocks = (nidx + rows_per_block - 1) / rows_per_block;
    if (block_dim) blocks = block_dim;
    if (blocks > 0x7fffffff) blocks = 0x7fffffff;
    AFIR_LAUNCH("gather_scale_shift_f16_vec", gather_scale_shift_f16_vec, dim3((unsigned)blocks), dim3(kThreads), 0,
                       stream, table, idx, scale, shift, out, error_flag, (uint32_t)rows, chunks,
                       nidx, lanes_per_row, rows_per_block);
  } else {
    int64_t blocks = (nidx + 3) / 4;
    if (block_dim) blocks = block_dim;
    if (blocks > 0x7fffffff) blocks = 0x7fffffff;
    AFIR_LAUNCH("gather_scale_shift_f16_any", gather_scale_shift_f16_any, dim3((unsigned)blocks), dim3(kThreads), 0,
                       stream, table, idx, scale, shift, out, error_flag, (uint32_t)rows, dim,
                       nidx);
  }
  return after_launch();
}

}  // namespace afir
