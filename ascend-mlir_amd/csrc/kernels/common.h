// Shared device helpers for the gfx950 fused kernels: 128-bit vector types,
// f16/bf16 <-> f32 conversion with one round-to-nearest-even, DPP wavefront
// reduction, and the host-side launch bookkeeping.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdlib.h>

namespace afir {

constexpr int kWave = 64;        // CDNA wavefront width
constexpr int kNumCU = 256;      // MI355X compute units (8 XCDs x 32): what the tile shapes were tuned on
constexpr int kNumXCD = 8;       // workgroup i runs on XCD i % 8; the matmul's tile order relies on it for
                                 // cache locality only (it is a permutation of the tiles whatever the part)

// Compute units of the device the process works on, asked once.  Grid sizes follow it, so a
// part with another CU count (a partitioned MI355X, say) gets grids of its own size; every
// kernel is grid-strided, so any value is correct.  kNumCU if the device cannot be asked.
inline int device_cus() {
  static const int count = [] {
    int device = 0, value = 0;
    if (hipGetDevice(&device) == hipSuccess &&
        hipDeviceGetAttribute(&value, hipDeviceAttributeMultiprocessorCount, device) == hipSuccess && value > 0)
      return value;
    (void)hipGetLastError();
    return kNumCU;
  }();
  return count;
}

// Read / write phase separation (the one-shot kernels of gather.hip and transpose.hip): a launch
// whose lanes are all resident at once requests everything it reads, holds its stores back
// until the chip's reads have been served, and then writes.  The hold is a time: ticks of the
// real-time counter the device reads with wall_clock64() (100 MHz on MI355X), counted from the
// start of each workgroup, base_ns + read_bytes / (gb_per_s GB/s).  AFIR_HIP_PHASED=0 in the
// environment switches the phased kernels off (the launchers then take their other kernels).
// (The default rates are those of the whole chip: a partition of it, with its share of the CUs,
// keeps to the other kernels unless AFIR_HIP_PHASED=1 says that the deployer has set the rates
// for it, the AFIR_*_PHASE_GBS variables below.)
inline bool phased_enabled() {
  const char *env = getenv("AFIR_HIP_PHASED");
  if (env && env[0] == '0') return false;
  return device_cus() == kNumCU || (env && env[0] == '1');
}
// A tuning constant that a deployer can change without rebuilding: the value of the environment
// variable `name` when it is set to an integer within [lo, hi], else `fallback` (the compile-time
// choice, which is what the tile searches found on a whole MI355X).  Read at every launch, so a
// search can step through values within one process.
inline int env_int(const char *name, int fallback, int lo, int hi) {
  const char *env = getenv(name);
  if (!env || !*env) return fallback;
  char *end = nullptr;
  const long v = strtol(env, &end, 10);
  return (end && *end == '\0' && v >= lo && v <= hi) ? (int)v : fallback;
}
// Workgroups of `kernel` that fit a compute unit at once, given its workgroup size and the
// dynamic LDS of the launch (registers and static LDS are the kernel's own): what a launch that
// wants all of its lanes resident together may count on.  0 if the runtime cannot say.
template <typename Kernel>
inline int resident_blocks_per_cu(Kernel kernel, int threads, size_t dynamic_lds) {
  int blocks = 0;
  if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&blocks, reinterpret_cast<const void *>(kernel), threads,
                                                   dynamic_lds) != hipSuccess) {
    (void)hipGetLastError();
    return 0;
  }
  return blocks;
}
inline int wall_clock_khz() {
  static const int khz = [] {
    int device = 0, value = 0;
    if (hipGetDevice(&device) == hipSuccess &&
        hipDeviceGetAttribute(&value, hipDeviceAttributeWallClockRate, device) == hipSuccess && value > 0)
      return value;
    (void)hipGetLastError();
    return 100000;
  }();
  return khz;
}
// A shape beyond the chip's resident lanes goes out as two phased launches of about equal size
// (the end of the first and the start of the second separate its writes from the other's reads):
// 3-7 % ahead of the unphased kernels at 96-128 MiB.  From three launches on the gaps between
// them cost what the separation gains (a 195 MiB gather: 3 % behind), so those shapes stay on
// the unphased kernels.
constexpr int kPhaseMaxLaunches = 2;
constexpr int kPhaseHoldMaxTicks = 1 << 14;      // ~164 us at 100 MHz: no launch waits longer than this
constexpr int kPhaseSpinLimit = 1 << 15;         // polls of the counter, whatever it reads
inline int phase_hold_ticks(int64_t read_bytes, int base_ns, int gb_per_s) {
  const double ns = (double)base_ns + (double)read_bytes / (double)gb_per_s;
  const double ticks = ns * 1e-6 * (double)wall_clock_khz();
  return ticks > (double)kPhaseHoldMaxTicks ? kPhaseHoldMaxTicks : (int)ticks;
}

// The hold of one workgroup of a phased launch, called once its own loads have arrived.  The
// chip serves the loads of a one-wave launch in the order of its workgroups (measured: the time
// from a workgroup's start to its last load grows linearly with blockIdx.x, 1.8 us for the first
// eighth of a 64 MiB copy, 8.7 us for the last), so a workgroup can tell from its own wait and its
// place in the launch when the last workgroup's loads will be back: latency + (wait - latency)
// * workgroups / (place + 1).  Alone that estimate is a poor hold (it overshoots for the early
// workgroups, whose small waits it multiplies most: 0.64-0.66 of peak against 0.75-0.78), but it
// is a good lower cut of the formula's: it falls under it when the reads run faster than the
// formula assumes (rows that repeat and come out of the caches, an input that still sits in the
// last-level cache), and then the workgroup waits only that long.  `below` is the fraction of the
// formula's hold under which the estimate is taken: with indices spread over the table every
// fraction from 0 (never) to 1 measures the same; with repeating rows 1 is the fastest (32768
// indices over 2048 rows: 23.2 us never, 17.0 at 1; the kernel without a hold 16.0).
constexpr int kPhaseLatencyTicks = 80;    // under every measured wait for a first load (0.9 us)
__device__ __forceinline__ int phase_hold_here(int hold_ticks, long long t_start, float below) {
  const int waited = (int)(wall_clock64() - t_start);
  const float over = waited > kPhaseLatencyTicks ? (float)(waited - kPhaseLatencyTicks) : 0.f;
  const float estimate = (float)kPhaseLatencyTicks + over * (float)gridDim.x / (float)(blockIdx.x + 1u);
  return estimate < below * (float)hold_ticks ? (int)estimate : hold_ticks;
}

// What the calling thread launched last: kernel, workgroups, lanes per workgroup.  A runner reads
// it back after a launcher call to report the grid the launcher chose (afir_hip_last_launch).
struct LaunchNote {
  const char *kernel;
  unsigned workgroups, threads;
};
inline LaunchNote &last_launch_note() {
  static thread_local LaunchNote note{"", 0u, 0u};
  return note;
}
#define AFIR_LAUNCH(name, kernel, grid, block, lds, stream, ...)                                     \
  do {                                                                                              \
    const dim3 afir_grid_ = (grid), afir_block_ = (block);                                          \
    ::afir::last_launch_note() = ::afir::LaunchNote{name, afir_grid_.x * afir_grid_.y * afir_grid_.z, \
                                                    afir_block_.x * afir_block_.y * afir_block_.z};  \
    hipLaunchKernelGGL(kernel, afir_grid_, afir_block_, lds, stream, __VA_ARGS__);                  \
  } while (0)

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

struct LaunchStatus {
  uint32_t code;
  const char *message;  // static string
};

// ---- storage conversions (device) -----------------------------------------

__device__ __forceinline__ float f16_lo(uint32_t packed) {
  return (float)__builtin_bit_cast(f16x2, packed).x;
}
__device__ __forceinline__ float f16_hi(uint32_t packed) {
  return (float)__builtin_bit_cast(f16x2, packed).y;
}
// two floats -> packed f16 pair, each rounded to nearest even
__device__ __forceinline__ uint32_t pack_f16(float lo, float hi) {
  f16x2 v;
  v.x = (_Float16)lo;
  v.y = (_Float16)hi;
  return __builtin_bit_cast(uint32_t, v);
}

__device__ __forceinline__ float bf16_lo(uint32_t packed) {
  return __uint_as_float(packed << 16);
}
__device__ __forceinline__ float bf16_hi(uint32_t packed) {
  return __uint_as_float(packed & 0xffff0000u);
}
__device__ __forceinline__ uint32_t f32_to_bf16_rne(float f) {
  uint32_t u = __float_as_uint(f);
  uint32_t r = (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
  // NaN: keep it a NaN after truncation
  return (f != f) ? ((u >> 16) | 0x40u) : r;
}
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
  return (f32_to_bf16_rne(lo) & 0xffffu) | (f32_to_bf16_rne(hi) << 16);
}
// The same two roundings in one instruction (v_cvt_pk_bf16_f32): bit-identical to pack_bf16 on
// every pair of non-NaN floats; a NaN stays a NaN (quiet bit set, top payload bits kept).
__device__ __forceinline__ uint32_t pack_bf16_hw(float lo, float hi) {
  typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
  typedef float f32x2_t __attribute__((ext_vector_type(2)));
  const f32x2_t v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}

// ---- wavefront reduction on DPP -------------------------------------------

template <int kCtrl>
__device__ __forceinline__ float dpp_add(float v) {
  int moved = __builtin_amdgcn_update_dpp(0, __float_as_int(v), kCtrl, 0xf, 0xf, true);
  return v + __int_as_float(moved);
}

// Sum over the 64 lanes; every lane returns the total.  Within a row of 16
// lanes: quad butterflies, then half-row and row mirrors; the four row totals
// are then read with readlane and added in a fixed order.
__device__ __forceinline__ float wave_sum(float v) {
  v = dpp_add<0xB1>(v);   // quad_perm [1,0,3,2]
  v = dpp_add<0x4E>(v);   // quad_perm [2,3,0,1]
  v = dpp_add<0x141>(v);  // row_half_mirror
  v = dpp_add<0x140>(v);  // row_mirror
  int iv = __float_as_int(v);
  float r0 = __int_as_float(__builtin_amdgcn_readlane(iv, 0));
  float r1 = __int_as_float(__builtin_amdgcn_readlane(iv, 16));
  float r2 = __int_as_float(__builtin_amdgcn_readlane(iv, 32));
  float r3 = __int_as_float(__builtin_amdgcn_readlane(iv, 48));
  return (r0 + r1) + (r2 + r3);
}

// ---- streaming memory access ------------------------------------------------

template <typename T>
__device__ __forceinline__ T load_nt(const T *p) {
#ifdef AFIR_PLAIN_LOADS
  return *p;
#else
  return __builtin_nontemporal_load(p);
#endif
}
template <typename T>
__device__ __forceinline__ void store_nt(T *p, T v) {
  __builtin_nontemporal_store(v, p);
}

__host__ inline bool aligned16(const void *p) {
  return (reinterpret_cast<uintptr_t>(p) & 15u) == 0;
}

}  // namespace afir
