// Generic fused-region kernel: executes a region program (postfix expression
// over affine-mapped input reads, optional row sum) for shapes and op chains
// that none of the hand-tuned kernels covers.  What the reference generates
// per region as AscendC source (parallel generics with Identity / broadcast /
// transposed / constant input maps and addf / mulf / maximumf bodies,
// lib/Conversion/LinalgToAscendC/ComputeConversion.cpp:1290-1640; reduction
// generics :246-750; the fused gather loop :828-1272) is here one interpreter
// whose program arrives as a kernel argument.
//
// HBM-bound by construction: a lane owns 8 consecutive elements of the
// innermost iteration dim, reads each operand once (128-bit loads where the
// operand is contiguous and aligned along that dim, one scalar load where it
// is broadcast along it, element loads for transposed or gathered operands),
// evaluates the chain in float32 registers and rounds once to the output
// type.  The program is wave-uniform (it lives in the kernel argument
// segment), so interpreting it costs scalar branches only; the value stack is
// four register vectors that are shifted on push and pop, which keeps every
// register index static.
#include "kernels.h"
#include "region_launch.h"

namespace afir {

namespace {

constexpr int kVec = 8;
constexpr int kThreads = 256;

__device__ __forceinline__ float load_elem(const void *base, int type, int64_t i) {
  if (type == kRegionF32) return static_cast<const float *>(base)[i];
  const uint32_t h = static_cast<const uint16_t *>(base)[i];
  if (type == kRegionF16) return (float)__builtin_bit_cast(_Float16, (uint16_t)h);
  return __uint_as_float(h << 16);
}

__device__ __forceinline__ void load_vec(const void *base, int type, int64_t i, float (&v)[kVec]) {
  if (type == kRegionF32) {
    const f32x4 *p = reinterpret_cast<const f32x4 *>(static_cast<const float *>(base) + i);
    const f32x4 a = p[0], b = p[1];
#pragma unroll
    for (int e = 0; e < 4; ++e) { v[e] = a[e]; v[4 + e] = b[e]; }
  } else {
    const u32x4 raw = *reinterpret_cast<const u32x4 *>(static_cast<const uint16_t *>(base) + i);
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      if (type == kRegionF16) { v[2 * d] = f16_lo(raw[d]); v[2 * d + 1] = f16_hi(raw[d]); }
      else { v[2 * d] = bf16_lo(raw[d]); v[2 * d + 1] = bf16_hi(raw[d]); }
    }
  }
}

__device__ __forceinline__ int64_t load_index(const void *base, int type, int64_t i) {
  return type == kRegionI32 ? (int64_t) static_cast<const int32_t *>(base)[i]
                            : static_cast<const int64_t *>(base)[i];
}

// One operand for the 8 elements j0..j0+7 of the innermost dim at outer
// position (i0, i1).  `full`: all 8 elements exist.
__device__ __forceinline__ void read_operand(const RegionInput &in, int last, int64_t i0,
                                             int64_t i1, int64_t j0, int nvalid, bool full,
                                             int32_t *error_flag, float (&v)[kVec]) {
  // iteration position of element j0: the innermost dim is `last`
  const int64_t x0 = last == 0 ? j0 : i0;
  const int64_t x1 = last == 1 ? j0 : i1;
  const int64_t x2 = last == 2 ? j0 : 0;
  // element position without the gathered dim
  const int64_t pos0 = in.offset + x0 * in.stride[0] + x1 * in.stride[1] + x2 * in.stride[2];
  int64_t pos = pos0;
  const int64_t step = last == 0 ? in.stride[0] : (last == 1 ? in.stride[1] : in.stride[2]);
  const float nan = __uint_as_float(0x7fc00000u);

  if (in.gdim < 0) {
    if (step == 1 && full && in.vec) {
      load_vec(in.base, in.type, pos, v);
    } else if (step == 0) {
      const float x = load_elem(in.base, in.type, pos);
#pragma unroll
      for (int e = 0; e < kVec; ++e) v[e] = x;
    } else {
#pragma unroll
      for (int e = 0; e < kVec; ++e) v[e] = (e < nvalid) ? load_elem(in.base, in.type, pos + e * step) : 0.f;
    }
    return;
  }
  if (in.gdim != last) {
    // the index is the same for the whole vector
    const int64_t g = load_index(in.index, in.gtype, in.gdim == 0 ? x0 : (in.gdim == 1 ? x1 : x2));
    if (g < 0 || g >= in.gextent) {
      if (error_flag) *error_flag = 1;
#pragma unroll
      for (int e = 0; e < kVec; ++e) v[e] = nan;
      return;
    }
    pos += g * in.gstride;
    if (step == 1 && full && in.vec && in.gvec) {
      load_vec(in.base, in.type, pos, v);
    } else if (step == 0) {
      const float x = load_elem(in.base, in.type, pos);
#pragma unroll
      for (int e = 0; e < kVec; ++e) v[e] = x;
    } else {
#pragma unroll
      for (int e = 0; e < kVec; ++e) v[e] = (e < nvalid) ? load_elem(in.base, in.type, pos + e * step) : 0.f;
    }
    return;
  }
  // gathered along the innermost dim: one index per element
#pragma unroll
  for (int e = 0; e < kVec; ++e) {
    float x = 0.f;
    if (e < nvalid) {
      const int64_t g = load_index(in.index, in.gtype, j0 + e);
      if (g < 0 || g >= in.gextent) {
        if (error_flag) *error_flag = 1;
        x = nan;
      } else {
        x = load_elem(in.base, in.type, pos + e * step + g * in.gstride);
      }
    }
    v[e] = x;
  }
}

// max / min with IEEE-754 maximum / minimum semantics (NaN propagates), as
// arith.maximumf / numpy.maximum define them.
__device__ __forceinline__ float fmax_nan(float a, float b) {
  return (a != a) ? a : ((b != b) ? b : ((a > b) ? a : ((b > a) ? b : ((__float_as_uint(a) & 0x80000000u) ? b : a))));
}
__device__ __forceinline__ float fmin_nan(float a, float b) {
  return (a != a) ? a : ((b != b) ? b : ((a < b) ? a : ((b < a) ? b : ((__float_as_uint(a) & 0x80000000u) ? a : b))));
}

// Evaluates the expression for 8 elements; the result is s0.
__device__ __forceinline__ void evaluate(const RegionArgs &R, int last, int64_t i0, int64_t i1,
                                         int64_t j0, int nvalid, bool full, float (&s0)[kVec]) {
  float s1[kVec], s2[kVec], s3[kVec];
#pragma unroll
  for (int e = 0; e < kVec; ++e) s0[e] = s1[e] = s2[e] = s3[e] = 0.f;
  auto push = [&]() {
#pragma unroll
    for (int e = 0; e < kVec; ++e) { s3[e] = s2[e]; s2[e] = s1[e]; s1[e] = s0[e]; }
  };
  auto pop_below = [&]() {  // drop s1, shifting the rest up
#pragma unroll
    for (int e = 0; e < kVec; ++e) { s1[e] = s2[e]; s2[e] = s3[e]; }
  };
  for (int pc = 0; pc < R.nops; ++pc) {
    const RegionOp op = R.ops[pc];
    switch (op.code) {
      case kRegionPush: {
        push();
        read_operand(R.in[op.input], last, i0, i1, j0, nvalid, full, R.error_flag, s0);
        break;
      }
      case kRegionConst:
        push();
#pragma unroll
        for (int e = 0; e < kVec; ++e) s0[e] = op.constant;
        break;
      case kRegionDup: {
        float t[kVec];
#pragma unroll
        for (int e = 0; e < kVec; ++e)
          t[e] = op.depth == 0 ? s0[e] : (op.depth == 1 ? s1[e] : (op.depth == 2 ? s2[e] : s3[e]));
        push();
#pragma unroll
        for (int e = 0; e < kVec; ++e) s0[e] = t[e];
        break;
      }
      case kRegionAdd:
#pragma unroll
        for (int e = 0; e < kVec; ++e) s0[e] = s1[e] + s0[e];
        pop_below();
        break;
      case kRegionSub:
#pragma unroll
        for (int e = 0; e < kVec; ++e) s0[e] = s1[e] - s0[e];
        pop_below();
        break;
      case kRegionMul:
#pragma unroll
        for (int e = 0; e < kVec; ++e) s0[e] = s1[e] * s0[e];
        pop_below();
        break;
      case kRegionDiv:
#pragma unroll
        for (int e = 0; e < kVec; ++e) s0[e] = s1[e] / s0[e];
        pop_below();
        break;
      case kRegionMax:
#pragma unroll
        for (int e = 0; e < kVec; ++e) s0[e] = fmax_nan(s1[e], s0[e]);
        pop_below();
        break;
      case kRegionMin:
#pragma unroll
        for (int e = 0; e < kVec; ++e) s0[e] = fmin_nan(s1[e], s0[e]);
        pop_below();
        break;
      case kRegionRelu:
#pragma unroll
        for (int e = 0; e < kVec; ++e) s0[e] = fmax_nan(s0[e], 0.f);
        break;
      case kRegionLeaky:
#pragma unroll
        for (int e = 0; e < kVec; ++e) s0[e] = fmax_nan(s0[e], s0[e] * op.constant);
        break;
      case kRegionNeg:
#pragma unroll
        for (int e = 0; e < kVec; ++e) s0[e] = -s0[e];
        break;
      default:
        break;
    }
  }
}

__device__ __forceinline__ void store_elem(void *out, int type, int64_t i, float x) {
  if (type == kRegionF32) static_cast<float *>(out)[i] = x;
  else if (type == kRegionF16) static_cast<uint16_t *>(out)[i] = __builtin_bit_cast(uint16_t, (_Float16)x);
  else static_cast<uint16_t *>(out)[i] = (uint16_t)f32_to_bf16_rne(x);
}

__global__ __launch_bounds__(kThreads) void fused_region_parallel(const RegionArgs R) {
  const int last = R.rank - 1;
  const int64_t n = R.size[last];
  const int64_t chunks = (n + kVec - 1) / kVec;
  const int64_t rows = (R.rank == 1) ? 1 : ((R.rank == 2) ? R.size[0] : R.size[0] * R.size[1]);
  const int64_t items = rows * chunks;
  const int64_t stride = (int64_t)gridDim.x * kThreads;
  for (int64_t item = (int64_t)blockIdx.x * kThreads + threadIdx.x; item < items; item += stride) {
    const int64_t row = item / chunks;
    const int64_t j0 = (item - row * chunks) * kVec;
    int64_t i0 = 0, i1 = 0;
    if (R.rank == 2) i0 = row;
    else if (R.rank == 3) { i0 = row / R.size[1]; i1 = row - i0 * R.size[1]; }
    const int64_t left = n - j0;
    const int nvalid = left >= kVec ? kVec : (int)left;
    const bool full = nvalid == kVec;
    float v[kVec];
    evaluate(R, last, i0, i1, j0, nvalid, full, v);
    const int64_t o = row * n + j0;
    if (full && R.out_vec) {
      if (R.out_type == kRegionF32) {
        f32x4 a, b;
#pragma unroll
        for (int e = 0; e < 4; ++e) { a[e] = v[e]; b[e] = v[4 + e]; }
        f32x4 *p = reinterpret_cast<f32x4 *>(static_cast<float *>(R.out) + o);
        p[0] = a;
        p[1] = b;
      } else {
        u32x4 w;
#pragma unroll
        for (int d = 0; d < 4; ++d)
          w[d] = R.out_type == kRegionF16 ? pack_f16(v[2 * d], v[2 * d + 1]) : pack_bf16(v[2 * d], v[2 * d + 1]);
        *reinterpret_cast<u32x4 *>(static_cast<uint16_t *>(R.out) + o) = w;
      }
    } else {
#pragma unroll
      for (int e = 0; e < kVec; ++e)
        if (e < nvalid) store_elem(R.out, R.out_type, o + e, v[e]);
    }
  }
}

// Row sum over the innermost dim: one wavefront per output element, lanes
// stride over the row in vectors of 8, float32 partial sums per vector slot,
// fixed-order combination and a DPP wave reduction: deterministic.
__global__ __launch_bounds__(kThreads) void fused_region_rowsum(const RegionArgs R) {
  const int last = R.rank - 1;
  const int64_t n = R.size[last];
  const int64_t chunks = (n + kVec - 1) / kVec;
  const int64_t rows = (R.rank == 2) ? R.size[0] : R.size[0] * R.size[1];
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t wave = (int64_t)blockIdx.x * (kThreads / kWave) + (threadIdx.x >> 6);
  const int64_t nwaves = (int64_t)gridDim.x * (kThreads / kWave);
  for (int64_t row = wave; row < rows; row += nwaves) {
    int64_t i0 = row, i1 = 0;
    if (R.rank == 3) { i0 = row / R.size[1]; i1 = row - i0 * R.size[1]; }
    float acc[kVec];
#pragma unroll
    for (int e = 0; e < kVec; ++e) acc[e] = 0.f;
    for (int64_t c = lane; c < chunks; c += kWave) {
      const int64_t j0 = c * kVec;
      const int64_t left = n - j0;
      const int nvalid = left >= kVec ? kVec : (int)left;
      float v[kVec];
      evaluate(R, last, i0, i1, j0, nvalid, nvalid == kVec, v);
#pragma unroll
      for (int e = 0; e < kVec; ++e) acc[e] += (e < nvalid) ? v[e] : 0.f;
    }
    float s = ((acc[0] + acc[1]) + (acc[2] + acc[3])) + ((acc[4] + acc[5]) + (acc[6] + acc[7]));
    s = wave_sum(s);
    if (lane == 0) store_elem(R.out, R.out_type, row, s);
  }
}

}  // namespace

LaunchStatus launch_fused_region(const RegionArgs &args, uint32_t block_dim, hipStream_t stream) {
  if (args.rank < 1 || args.rank > 3) return invalid("fused_region: bad iteration rank");
  if (args.nops < 0 || args.nops > kRegionMaxOps || args.ninputs < 0 || args.ninputs > kRegionMaxInputs)
    return invalid("fused_region: program too large");
  int64_t rows = 1, total = 1;
  for (int k = 0; k < args.rank; ++k) {
    if (args.size[k] < 0) return invalid("fused_region: negative extent");
    if (args.size[k] != 0 && total > INT64_MAX / 16 / args.size[k]) return invalid("fused_region: extent overflow");
    total *= args.size[k];
    if (k + 1 < args.rank) rows *= args.size[k];
  }
  if (args.reduce) {
    if (args.rank < 2) return invalid("fused_region: reduction needs rank >= 2");
    if (rows == 0) return ok_status();
    if (!args.out) return invalid("fused_region: null output pointer");
    int64_t blocks = (rows + (kThreads / kWave) - 1) / (kThreads / kWave);
    if (blocks > (int64_t)kNumCU * 8) blocks = (int64_t)kNumCU * 8;
    if (block_dim) blocks = block_dim;
    hipLaunchKernelGGL(fused_region_rowsum, dim3((unsigned)blocks), dim3(kThreads), 0, stream, args);
    return after_launch();
  }
  if (total == 0) return ok_status();
  if (!args.out) return invalid("fused_region: null output pointer");
  const int64_t n = args.size[args.rank - 1];
  const int64_t items = rows * ((n + kVec - 1) / kVec);
  int64_t blocks = (items + kThreads - 1) / kThreads;
  if (blocks > (int64_t)kNumCU * 16) blocks = (int64_t)kNumCU * 16;
  if (block_dim) blocks = block_dim;
  hipLaunchKernelGGL(fused_region_parallel, dim3((unsigned)blocks), dim3(kThreads), 0, stream, args);
  return after_launch();
}

}  // namespace afir
