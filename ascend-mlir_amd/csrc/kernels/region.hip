// Generic fused-region kernel: executes a region program (postfix expression
// over affine-mapped input reads, optional row sum) for shapes and op chains
// that none of the hand-tuned kernels covers.  What the reference generates
// per region as AscendC source (parallel generics with Identity / broadcast /
// transposed / constant input maps and addf / mulf / maximumf bodies,
// lib/Conversion/LinalgToAscendC/ComputeConversion.cpp:1290-1640; reduction
// generics :246-750; the fused gather loop :828-1272) is here one interpreter
// whose program arrives as a kernel argument.
//
// HBM-bound by construction: a lane owns 8 (or 16) consecutive elements of the
// innermost iteration dim, reads each operand once (128-bit loads where the
// operand is contiguous and aligned along that dim, one scalar load where it
// is broadcast along it, element loads for transposed or gathered operands),
// evaluates the chain in float32 registers and rounds once to the output
// type.  The program is wave-uniform (it lives in the kernel argument
// segment), so interpreting it costs scalar branches only.  The value stack is
// four register vectors; the launcher resolves every operation's stack slot on
// the host, so the kernel never shifts the stack: an operation is a scalar
// switch on its slot and then straight-line vector code.  Rows and 8-element
// chunks are assigned to lanes without a division (a row of at most 256
// chunks takes a power-of-two group of lanes, longer rows take the whole
// workgroup), and positions are 32-bit when every tensor is below 2^31
// elements.
//
// Most fused regions are chains -- a running value combined with one new
// operand per step, activations in between (every example graph of the
// reference is one).  The launcher recognises that shape and hands the kernel
// the linear form: one accumulator vector and one operand vector are the only
// live values, no stack and no moves, which leaves registers for eight waves
// per SIMD.  Expressions that are not chains run on the stack interpreter.
#include <cstdlib>

#include "kernels.h"
#include "region_launch.h"

namespace afir {

namespace {

constexpr int kThreads = 256;

__device__ __forceinline__ float load_elem(const void *base, int type, int64_t i) {
  if (type == kRegionF32 || type == kRegionI32) return static_cast<const float *>(base)[i];   // i32: the bits
  if (type == kRegionI16) return __int_as_float((int)static_cast<const int16_t *>(base)[i]);
  const uint32_t h = static_cast<const uint16_t *>(base)[i];
  if (type == kRegionF16) return (float)__builtin_bit_cast(_Float16, (uint16_t)h);
  return __uint_as_float(h << 16);
}

template <int V>
__device__ __forceinline__ void load_vec(const void *base, int type, int64_t i, float (&v)[V]) {
  if (type == kRegionF32 || type == kRegionI32) {
    const f32x4 *p = reinterpret_cast<const f32x4 *>(static_cast<const float *>(base) + i);
#pragma unroll
    for (int q = 0; q < V / 4; ++q) {
      const f32x4 a = p[q];
#pragma unroll
      for (int e = 0; e < 4; ++e) v[4 * q + e] = a[e];
    }
  } else {
    const u32x4 *p = reinterpret_cast<const u32x4 *>(static_cast<const uint16_t *>(base) + i);
#pragma unroll
    for (int q = 0; q < V / 8; ++q) {
      const u32x4 raw = p[q];
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        if (type == kRegionF16) { v[8 * q + 2 * d] = f16_lo(raw[d]); v[8 * q + 2 * d + 1] = f16_hi(raw[d]); }
        else if (type == kRegionI16) {   // sign-extended
          v[8 * q + 2 * d] = __int_as_float((int)(raw[d] << 16) >> 16);
          v[8 * q + 2 * d + 1] = __int_as_float((int)raw[d] >> 16);
        }
        else { v[8 * q + 2 * d] = bf16_lo(raw[d]); v[8 * q + 2 * d + 1] = bf16_hi(raw[d]); }
      }
    }
  }
}

__device__ __forceinline__ int64_t load_index(const void *base, int type, int64_t i) {
  return type == kRegionI32 ? (int64_t) static_cast<const int32_t *>(base)[i]
                            : static_cast<const int64_t *>(base)[i];
}

// Iteration position of the first of a lane's V elements.
template <typename I>
struct Position {
  I x0, x1, x2;  // index along iteration dims 0..2 (the innermost one holds j0)
};

// One operand for the V elements at `at`.  `full`: all V elements exist.
template <typename I, int V>
__device__ __forceinline__ void read_operand(const RegionInput &in, int last, const Position<I> &at,
                                             int nvalid, bool full, int32_t *error_flag,
                                             float (&v)[V]) {
  // element position without the gathered dim
  I pos = (I)in.offset + at.x0 * (I)in.stride[0] + at.x1 * (I)in.stride[1] + at.x2 * (I)in.stride[2];
  const I step = (I)(last == 0 ? in.stride[0] : (last == 1 ? in.stride[1] : in.stride[2]));
  // what an out-of-range gather yields: NaN, or 0 in an integer region
  const float nan = (in.type == kRegionI32 || in.type == kRegionI16) ? 0.f : __uint_as_float(0x7fc00000u);

  if (in.gdim >= 0 && in.gdim == last) {
    // gathered along the innermost dim: one index per element
    const I j0 = last == 0 ? at.x0 : (last == 1 ? at.x1 : at.x2);
#pragma unroll
    for (int e = 0; e < V; ++e) {
      float x = 0.f;
      if (e < nvalid) {
        const int64_t g = load_index(in.index, in.gtype, (int64_t)j0 + e);
        if (g < 0 || g >= in.gextent) {
          if (error_flag) *error_flag = 1;
          x = nan;
        } else {
          x = load_elem(in.base, in.type, (int64_t)pos + (int64_t)e * step + g * in.gstride);
        }
      }
      v[e] = x;
    }
    return;
  }
  bool vec = in.vec != 0;
  int64_t p64 = (int64_t)pos;
  if (in.gdim >= 0) {
    // the index is the same for the whole vector
    const int64_t g = load_index(in.index, in.gtype,
                                 (int64_t)(in.gdim == 0 ? at.x0 : (in.gdim == 1 ? at.x1 : at.x2)));
    if (g < 0 || g >= in.gextent) {
      if (error_flag) *error_flag = 1;
#pragma unroll
      for (int e = 0; e < V; ++e) v[e] = nan;
      return;
    }
    p64 += g * in.gstride;
    vec = vec && in.gvec;
  }
  if (step == 1 && full && vec) {
    load_vec(in.base, in.type, p64, v);
  } else if (step == 0) {
    const float x = load_elem(in.base, in.type, p64);
#pragma unroll
    for (int e = 0; e < V; ++e) v[e] = x;
  } else {
#pragma unroll
    for (int e = 0; e < V; ++e)
      v[e] = (e < nvalid) ? load_elem(in.base, in.type, p64 + (int64_t)e * step) : 0.f;
  }
}

// max / min with IEEE-754 maximum / minimum semantics (NaN propagates, -0 < +0),
// as arith.maximumf / arith.minimumf define them: v_maximum3_f32 / v_minimum3_f32.
__device__ __forceinline__ float fmax_nan(float a, float b) { return __builtin_elementwise_maximum(a, b); }
__device__ __forceinline__ float fmin_nan(float a, float b) { return __builtin_elementwise_minimum(a, b); }

// Every operation has its own case and the default does nothing: with the
// last operation as the default, hipcc 7.2 lost the eighth element of a
// negation that followed a binary step in the chain evaluator.
template <int V>
__device__ __forceinline__ void binary(int code, float (&a)[V], const float (&b)[V]) {
  switch (code) {
    case kRegionAdd:
#pragma unroll
      for (int e = 0; e < V; ++e) a[e] = a[e] + b[e];
      break;
    case kRegionSub:
#pragma unroll
      for (int e = 0; e < V; ++e) a[e] = a[e] - b[e];
      break;
    case kRegionMul:
#pragma unroll
      for (int e = 0; e < V; ++e) a[e] = a[e] * b[e];
      break;
    case kRegionDiv:
#pragma unroll
      for (int e = 0; e < V; ++e) a[e] = a[e] / b[e];
      break;
    case kRegionMax:
#pragma unroll
      for (int e = 0; e < V; ++e) a[e] = fmax_nan(a[e], b[e]);
      break;
    case kRegionMin:
#pragma unroll
      for (int e = 0; e < V; ++e) a[e] = fmin_nan(a[e], b[e]);
      break;
    // 32-bit two's complement, wrapping (unsigned arithmetic)
    case kRegionAddI:
#pragma unroll
      for (int e = 0; e < V; ++e) a[e] = __uint_as_float(__float_as_uint(a[e]) + __float_as_uint(b[e]));
      break;
    case kRegionSubI:
#pragma unroll
      for (int e = 0; e < V; ++e) a[e] = __uint_as_float(__float_as_uint(a[e]) - __float_as_uint(b[e]));
      break;
    case kRegionMulI:
#pragma unroll
      for (int e = 0; e < V; ++e) a[e] = __uint_as_float(__float_as_uint(a[e]) * __float_as_uint(b[e]));
      break;
    case kRegionMaxI:
#pragma unroll
      for (int e = 0; e < V; ++e) a[e] = __float_as_int(a[e]) > __float_as_int(b[e]) ? a[e] : b[e];
      break;
    case kRegionMinI:
#pragma unroll
      for (int e = 0; e < V; ++e) a[e] = __float_as_int(a[e]) < __float_as_int(b[e]) ? a[e] : b[e];
      break;
    case kRegionMaxI16:
#pragma unroll
      for (int e = 0; e < V; ++e) {
        const int x = (short)__float_as_int(a[e]), y = (short)__float_as_int(b[e]);
        a[e] = __int_as_float(x > y ? x : y);
      }
      break;
    case kRegionMinI16:
#pragma unroll
      for (int e = 0; e < V; ++e) {
        const int x = (short)__float_as_int(a[e]), y = (short)__float_as_int(b[e]);
        a[e] = __int_as_float(x < y ? x : y);
      }
      break;
    default:
      break;
  }
}

template <int V>
__device__ __forceinline__ void unary(int code, float c, float (&a)[V]) {
  switch (code) {
    case kRegionRelu:
#pragma unroll
      for (int e = 0; e < V; ++e) a[e] = fmax_nan(a[e], 0.f);
      break;
    case kRegionLeaky:
#pragma unroll
      for (int e = 0; e < V; ++e) a[e] = fmax_nan(a[e], a[e] * c);
      break;
    case kRegionNeg:
#pragma unroll
      for (int e = 0; e < V; ++e) a[e] = -a[e];
      break;
    case kRegionCastF16:
#pragma unroll
      for (int e = 0; e < V; ++e) a[e] = (float)(_Float16)a[e];
      break;
    case kRegionCastBF16:
#pragma unroll
      for (int e = 0; e < V; ++e) a[e] = __uint_as_float(f32_to_bf16_rne(a[e]) << 16);
      break;
    case kRegionReluI:
#pragma unroll
      for (int e = 0; e < V; ++e) a[e] = __float_as_int(a[e]) > 0 ? a[e] : 0.f;
      break;
    case kRegionNegI:
#pragma unroll
      for (int e = 0; e < V; ++e) a[e] = __uint_as_float(0u - __float_as_uint(a[e]));
      break;
    case kRegionReluI16:
#pragma unroll
      for (int e = 0; e < V; ++e) {
        const int x = (short)__float_as_int(a[e]);
        a[e] = __int_as_float(x > 0 ? x : 0);
      }
      break;
    default:
      break;
  }
}

template <int V>
__device__ __forceinline__ void assign(float (&d)[V], const float (&s)[V]) {
#pragma unroll
  for (int e = 0; e < V; ++e) d[e] = s[e];
}

// Evaluates the expression for V elements; the result ends up in slot 0.
template <typename I, int V>
__device__ __forceinline__ void evaluate(const RegionArgs &R, int last, const Position<I> &at,
                                         int nvalid, bool full, float (&s0)[V]) {
  float s1[V], s2[V], s3[V];
#pragma unroll
  for (int e = 0; e < V; ++e) s0[e] = s1[e] = s2[e] = s3[e] = 0.f;
  for (int pc = 0; pc < R.nops; ++pc) {
    const RegionOp op = R.ops[pc];
    if (op.code == kRegionPush || op.code == kRegionConst || op.code == kRegionDup) {
      float t[V];
      if (op.code == kRegionPush) {
        read_operand<I, V>(R.in[op.input], last, at, nvalid, full, R.error_flag, t);
      } else if (op.code == kRegionConst) {
#pragma unroll
        for (int e = 0; e < V; ++e) t[e] = op.constant;
      } else {
        const int src = op.dst - 1 - op.depth;
        assign(t, src == 0 ? s0 : (src == 1 ? s1 : s2));
      }
      switch (op.dst) {
        case 0: assign(s0, t); break;
        case 1: assign(s1, t); break;
        case 2: assign(s2, t); break;
        default: assign(s3, t); break;
      }
    } else if (region_is_binary(op.code)) {   // binary: slot dst (op) slot dst + 1
      switch (op.dst) {
        case 0: binary(op.code, s0, s1); break;
        case 1: binary(op.code, s1, s2); break;
        default: binary(op.code, s2, s3); break;
      }
    } else {
      switch (op.dst) {
        case 0: unary(op.code, op.constant, s0); break;
        case 1: unary(op.code, op.constant, s1); break;
        case 2: unary(op.code, op.constant, s2); break;
        default: unary(op.code, op.constant, s3); break;
      }
    }
  }
}

template <int V>
__device__ __forceinline__ void apply_unaries(const RegionUnary &u, float (&a)[V]) {
  if (u.count > 0) unary(u.code[0], u.alpha[0], a);
  if (u.count > 1) unary(u.code[1], u.alpha[1], a);
}

// Linear form: acc = u0(x0); acc = u_k(acc (op_k) x_k).
template <typename I, int V>
__device__ __forceinline__ void evaluate_chain(const RegionArgs &R, int last, const Position<I> &at,
                                               int nvalid, bool full, float (&acc)[V]) {
  if (R.chain_first >= 0) {
    read_operand<I, V>(R.in[R.chain_first], last, at, nvalid, full, R.error_flag, acc);
  } else {
#pragma unroll
    for (int e = 0; e < V; ++e) acc[e] = R.chain_constant;
  }
  apply_unaries(R.chain_after_first, acc);
  for (int k = 0; k < R.nsteps; ++k) {
    const RegionStep &st = R.steps[k];
    float x[V];
    if (st.input >= 0) {
      read_operand<I, V>(R.in[st.input], last, at, nvalid, full, R.error_flag, x);
    } else {
#pragma unroll
      for (int e = 0; e < V; ++e) x[e] = st.constant;
    }
    if (st.bop == kChainRSub) {
#pragma unroll
      for (int e = 0; e < V; ++e) acc[e] = x[e] - acc[e];
    } else if (st.bop == kChainRDiv) {
#pragma unroll
      for (int e = 0; e < V; ++e) acc[e] = x[e] / acc[e];
    } else if (st.bop == kChainRSubI) {
#pragma unroll
      for (int e = 0; e < V; ++e) acc[e] = __uint_as_float(__float_as_uint(x[e]) - __float_as_uint(acc[e]));
    } else {
      binary(st.bop, acc, x);
    }
    apply_unaries(st.after, acc);
  }
}

template <typename I, bool CHAIN, int V>
__device__ __forceinline__ void evaluate_any(const RegionArgs &R, int last, const Position<I> &at,
                                             int nvalid, bool full, float (&v)[V]) {
  if (CHAIN) evaluate_chain<I, V>(R, last, at, nvalid, full, v);
  else evaluate<I, V>(R, last, at, nvalid, full, v);
}

__device__ __forceinline__ void store_elem(void *out, int type, int64_t i, float x) {
  if (type == kRegionF32 || type == kRegionI32) static_cast<float *>(out)[i] = x;   // i32: the bits
  else if (type == kRegionI16) static_cast<uint16_t *>(out)[i] = (uint16_t)__float_as_uint(x);
  else if (type == kRegionF16) static_cast<uint16_t *>(out)[i] = __builtin_bit_cast(uint16_t, (_Float16)x);
  else static_cast<uint16_t *>(out)[i] = (uint16_t)f32_to_bf16_rne(x);
}

template <typename I>
__device__ __forceinline__ Position<I> position(const RegionArgs &R, I row, I j0) {
  Position<I> p;
  if (R.rank == 1) { p.x0 = j0; p.x1 = 0; p.x2 = 0; }
  else if (R.rank == 2) { p.x0 = row; p.x1 = j0; p.x2 = 0; }
  else {
    // unsigned 32-bit division where it fits: an order of magnitude cheaper
    // than the 64-bit one
    if (sizeof(I) == 4) p.x0 = (I)((uint32_t)row / (uint32_t)R.size[1]);
    else p.x0 = row / (I)R.size[1];
    p.x1 = row - p.x0 * (I)R.size[1];
    p.x2 = j0;
  }
  return p;
}

// lanes_log2: a row's chunks are spread over 2^lanes_log2 lanes of the
// workgroup (8 = the whole workgroup walks one row at a time).
template <typename I, bool CHAIN, int V>
__global__ __launch_bounds__(kThreads) void fused_region_parallel(const RegionArgs R, int lanes_log2) {
  const int last = R.rank - 1;
  const I n = (I)R.size[last];
  const I chunks = (n + V - 1) / V;
  const I rows = (I)((R.rank == 1) ? 1 : ((R.rank == 2) ? R.size[0] : R.size[0] * R.size[1]));
  const int lanes = 1 << lanes_log2;
  const int rows_per_pass = kThreads >> lanes_log2;
  const I local_row = (I)(threadIdx.x >> lanes_log2);
  const I first_chunk = (I)(threadIdx.x & (lanes - 1));
  // blockIdx.y: which stretches of a long row this workgroup takes (few, long rows
  // are spread over workgroups along the row as well)
  for (I row0 = (I)blockIdx.x * rows_per_pass; row0 < rows; row0 += (I)gridDim.x * rows_per_pass) {
    const I row = row0 + local_row;
    if (row >= rows) continue;
    for (I chunk = first_chunk + (I)blockIdx.y * lanes; chunk < chunks; chunk += (I)gridDim.y * lanes) {
      const I j0 = chunk * V;
      const I left = n - j0;
      const int nvalid = left >= V ? V : (int)left;
      const bool full = nvalid == V;
      float v[V];
      evaluate_any<I, CHAIN, V>(R, last, position<I>(R, row, j0), nvalid, full, v);
      const int64_t o = (int64_t)row * n + j0;
      if (full && R.out_vec) {
        if (R.out_type == kRegionF32 || R.out_type == kRegionI32) {
          f32x4 *p = reinterpret_cast<f32x4 *>(static_cast<float *>(R.out) + o);
#pragma unroll
          for (int q = 0; q < V / 4; ++q) {
            f32x4 a;
#pragma unroll
            for (int e = 0; e < 4; ++e) a[e] = v[4 * q + e];
            p[q] = a;
          }
        } else {
          u32x4 *p = reinterpret_cast<u32x4 *>(static_cast<uint16_t *>(R.out) + o);
#pragma unroll
          for (int q = 0; q < V / 8; ++q) {
            u32x4 w;
#pragma unroll
            for (int d = 0; d < 4; ++d)
              w[d] = R.out_type == kRegionF16 ? pack_f16(v[8 * q + 2 * d], v[8 * q + 2 * d + 1])
                     : R.out_type == kRegionI16
                         ? ((__float_as_uint(v[8 * q + 2 * d]) & 0xffffu) | (__float_as_uint(v[8 * q + 2 * d + 1]) << 16))
                         : pack_bf16(v[8 * q + 2 * d], v[8 * q + 2 * d + 1]);
            p[q] = w;
          }
        }
      } else {
#pragma unroll
        for (int e = 0; e < V; ++e)
          if (e < nvalid) store_elem(R.out, R.out_type, o + e, v[e]);
      }
    }
  }
}

// What a reduce segment does to a row's sum before storing it (mean = sum / N, ...).
__device__ __forceinline__ float apply_tail(const RegionArgs &R, float s) {
  for (int k = 0; k < R.ntail; ++k) {
    const RegionOp &op = R.tail[k];
    float a[1] = {op.depth ? op.constant : s};
    const float b[1] = {op.depth ? s : op.constant};
    if (region_is_binary(op.code)) binary<1>(op.code, a, b);
    else unary<1>(op.code, op.constant, a);
    s = a[0];
  }
  return s;
}

// Row sum over the innermost dim: 2^lanes_log2 lanes of a wavefront per output
// element (the whole wavefront for rows of 64 vectors or more, fewer lanes and
// several rows per wavefront for shorter rows), the lanes stride over the row in
// vectors of V, float32 partial sums per vector slot, fixed-order combination
// and a DPP wave reduction or a butterfly over the row's lanes: deterministic.
template <typename I, bool CHAIN, int V>
__global__ __launch_bounds__(kThreads) void fused_region_rowsum(const RegionArgs R, int lanes_log2) {
  const int last = R.rank - 1;
  const I n = (I)R.size[last];
  const I chunks = (n + V - 1) / V;
  const I rows = (I)((R.rank == 2) ? R.size[0] : R.size[0] * R.size[1]);
  const int lane = threadIdx.x & (kWave - 1);
  const int lanes = 1 << lanes_log2;
  const I rows_per_wave = (I)(kWave >> lanes_log2);
  const I wave = (I)blockIdx.x * (kThreads / kWave) + (I)(threadIdx.x >> 6);
  const I nwaves = (I)gridDim.x * (kThreads / kWave);
  for (I row0 = wave * rows_per_wave; row0 < rows; row0 += nwaves * rows_per_wave) {
    const I row = row0 + (I)(lane >> lanes_log2);
    if (row >= rows) continue;   // the lanes of a row leave together
    float acc[V];
#pragma unroll
    for (int e = 0; e < V; ++e) acc[e] = 0.f;
    for (I c = lane & (lanes - 1); c < chunks; c += lanes) {
      const I j0 = c * V;
      const I left = n - j0;
      const int nvalid = left >= V ? V : (int)left;
      float v[V];
      evaluate_any<I, CHAIN, V>(R, last, position<I>(R, row, j0), nvalid, nvalid == V, v);
#pragma unroll
      for (int e = 0; e < V; ++e) acc[e] += (e < nvalid) ? v[e] : 0.f;
    }
    // fixed-order pairwise combination of the per-slot partial sums
#pragma unroll
    for (int w = V / 2; w >= 1; w >>= 1)
#pragma unroll
      for (int e = 0; e < w; ++e) acc[e] = acc[2 * e] + acc[2 * e + 1];
    float s = acc[0];
    if (lanes_log2 == 6) {
      s = wave_sum(s);
    } else {
      for (int m = lanes >> 1; m >= 1; m >>= 1) s += __shfl_xor(s, m);
    }
    if ((lane & (lanes - 1)) == 0) store_elem(R.out, R.out_type, (int64_t)row, apply_tail(R, s));
  }
}

// Postfix program -> linear chain, where the expression is one: at most one
// partial result is alive at any time and every other stack entry is a leaf
// (an operand read or a constant, with activations only on the leaf the chain
// starts from).  Returns false for anything else (two partial results, dup).
bool linearize(RegionArgs &a) {
  struct Entry {
    bool chain = false;
    int input = -1;          // leaf: operand, or -1 = constant
    float constant = 0.f;
    RegionUnary un = {};
  };
  Entry stack[4];
  int depth = 0;
  bool started = false;
  a.nsteps = 0;
  a.chain_after_first = RegionUnary{};
  auto reversed = [](int code) {
    return code == kRegionSub ? (int)kChainRSub
                              : (code == kRegionDiv ? (int)kChainRDiv : (code == kRegionSubI ? (int)kChainRSubI : code));
  };
  auto add_unary = [](RegionUnary &u, int code, float alpha) {
    if (u.count >= 2) return false;
    u.code[u.count] = code;
    u.alpha[u.count] = alpha;
    ++u.count;
    return true;
  };
  auto add_step = [&](int bop, const Entry &leaf) {
    if (a.nsteps >= kRegionMaxSteps) return false;
    RegionStep &st = a.steps[a.nsteps++];
    st = RegionStep{};
    st.bop = bop;
    st.input = leaf.input;
    st.constant = leaf.constant;
    return true;
  };
  auto start = [&](const Entry &leaf) {
    started = true;
    a.chain_first = leaf.input;
    a.chain_constant = leaf.constant;
    a.chain_after_first = leaf.un;
  };
  for (int i = 0; i < a.nops; ++i) {
    const RegionOp &op = a.ops[i];
    if (op.code == kRegionPush || op.code == kRegionConst) {
      Entry e;
      e.input = op.code == kRegionPush ? op.input : -1;
      e.constant = op.constant;
      stack[depth++] = e;
    } else if (op.code == kRegionDup) {
      return false;
    } else if (region_is_binary(op.code)) {
      Entry &x = stack[depth - 2], &y = stack[depth - 1];
      if (x.chain && y.chain) return false;
      if (x.chain) {
        if (y.un.count || !add_step(op.code, y)) return false;
      } else if (y.chain) {
        if (x.un.count || !add_step(reversed(op.code), x)) return false;
        x = y;
      } else {
        if (started) return false;          // a second partial result
        if (x.un.count && y.un.count) return false;
        if (y.un.count) {
          start(y);
          if (!add_step(reversed(op.code), x)) return false;
        } else {
          start(x);
          if (!add_step(op.code, y)) return false;
        }
        x = Entry{};
        x.chain = true;
      }
      --depth;
    } else {   // unary
      Entry &x = stack[depth - 1];
      RegionUnary &u = x.chain ? (a.nsteps ? a.steps[a.nsteps - 1].after : a.chain_after_first) : x.un;
      if (!add_unary(u, op.code, op.constant)) return false;
    }
  }
  if (!stack[0].chain) {   // a single leaf: x0 with its activations, no steps
    if (started) return false;
    start(stack[0]);
  }
  return true;
}

}  // namespace

LaunchStatus plan_fused_region(const RegionArgs &args, int vec, uint32_t block_dim, RegionGeometry *g) {
  if (args.rank < 1 || args.rank > 3) return invalid("fused_region: bad iteration rank");
  if (args.ninputs < 0 || args.ninputs > kRegionMaxInputs) return invalid("fused_region: program too large");
  int64_t rows = 1, total = 1;
  for (int k = 0; k < args.rank; ++k) {
    if (args.size[k] < 0) return invalid("fused_region: negative extent");
    if (args.size[k] != 0 && total > INT64_MAX / 16 / args.size[k]) return invalid("fused_region: extent overflow");
    total *= args.size[k];
    if (k + 1 < args.rank) rows *= args.size[k];
  }
  // 32-bit positions when every operand and the output stay below 2^31 elements
  // (with room for the positions of a last, partly empty pass)
  bool idx32 = total < ((int64_t)1 << 31) - 65536;
  for (int i = 0; i < args.ninputs && idx32; ++i) {
    int64_t reach = args.in[i].offset < 0 ? -args.in[i].offset : args.in[i].offset;
    for (int k = 0; k < args.rank; ++k) {
      const int64_t st = args.in[i].stride[k] < 0 ? -args.in[i].stride[k] : args.in[i].stride[k];
      if (args.size[k] > 0 && st > (((int64_t)1 << 31) - 1 - reach) / args.size[k]) { idx32 = false; break; }
      reach += st * (args.size[k] > 0 ? args.size[k] - 1 : 0);
    }
  }
  g->idx32 = idx32;
  g->lanes_log2 = 0;
  g->blocks = 0;
  if (args.reduce) {
    if (args.rank < 2) return invalid("fused_region: reduction needs rank >= 2");
    g->empty = rows == 0;
    if (g->empty) return ok_status();
    if (!args.out) return invalid("fused_region: null output pointer");
    // lanes of a wavefront that share a row: enough to cover a short row in one pass
    const int64_t row_chunks = (args.size[args.rank - 1] + vec - 1) / vec;
    int ll = 0;
    while (ll < 6 && ((int64_t)1 << ll) < row_chunks) ++ll;
    const int64_t rows_per_block = (int64_t)(kThreads / kWave) * (kWave >> ll);
    int64_t blocks = (rows + rows_per_block - 1) / rows_per_block;
    // up to 64 waves per CU at a time; 16 and more measured 3 % above 8 on 16384 rows of f16
    if (blocks > (int64_t)device_cus() * 16) blocks = (int64_t)device_cus() * 16;
    if (block_dim) blocks = block_dim;
    g->blocks = blocks;
    g->lanes_log2 = ll;
    return ok_status();
  }
  g->empty = total == 0;
  if (g->empty) return ok_status();
  if (!args.out) return invalid("fused_region: null output pointer");
  const int64_t n = args.size[args.rank - 1];
  const int64_t chunks = (n + vec - 1) / vec;
  int lanes_log2 = 0;
  while (lanes_log2 < 8 && ((int64_t)1 << lanes_log2) < chunks) ++lanes_log2;
  const int rows_per_pass = kThreads >> lanes_log2;
  int64_t blocks = (rows + rows_per_pass - 1) / rows_per_pass;
  if (blocks > (int64_t)device_cus() * 16) blocks = (int64_t)device_cus() * 16;
  // few rows that are longer than one pass of the workgroup: more workgroups along the row
  const int64_t passes = (chunks + ((int64_t)1 << lanes_log2) - 1) >> lanes_log2;
  int64_t column_blocks = (int64_t)device_cus() * 16 / blocks;
  if (column_blocks > passes) column_blocks = passes;
  if (column_blocks > 65535) column_blocks = 65535;
  if (column_blocks < 1) column_blocks = 1;
  if (block_dim) {
    blocks = block_dim;
    column_blocks = 1;
  }
  g->blocks = blocks * column_blocks;
  g->column_blocks = column_blocks;
  g->lanes_log2 = lanes_log2;
  return ok_status();
}

LaunchStatus launch_fused_region(const RegionArgs &args_in, uint32_t block_dim, hipStream_t stream) {
  RegionArgs args = args_in;
  if (args.rank < 1 || args.rank > 3) return invalid("fused_region: bad iteration rank");
  if (args.nops < 0 || args.nops > kRegionMaxOps || args.ninputs < 0 || args.ninputs > kRegionMaxInputs)
    return invalid("fused_region: program too large");
  // stack slots: the interpreter does not shift values, every operation is
  // told where its operands live
  int depth = 0;
  for (int i = 0; i < args.nops; ++i) {
    RegionOp &op = args.ops[i];
    if (op.code == kRegionPush || op.code == kRegionConst || op.code == kRegionDup) {
      if (op.code == kRegionDup && (op.depth < 0 || op.depth >= depth)) return invalid("fused_region: dup beyond the stack");
      op.dst = depth++;
      if (depth > 4) return invalid("fused_region: more than 4 live values");
      if (op.code == kRegionPush && (op.input < 0 || op.input >= args.ninputs)) return invalid("fused_region: bad operand");
    } else if (region_is_binary(op.code)) {
      if (depth < 2) return invalid("fused_region: binary operation on fewer than two values");
      op.dst = depth - 2;
      --depth;
    } else if (region_is_unary(op.code)) {
      if (depth < 1) return invalid("fused_region: unary operation on an empty stack");
      op.dst = depth - 1;
    } else {
      return invalid("fused_region: unknown operation code");
    }
  }
  if (depth != 1) return invalid("fused_region: the program must leave exactly one value");
  args.chain = linearize(args) ? 1 : 0;
  // AFIR_HIP_REGION_STACK=1 keeps chains on the stack interpreter (the tests
  // run every program both ways)
  if (const char *env = std::getenv("AFIR_HIP_REGION_STACK"))
    if (*env && *env != '0') args.chain = 0;

  // 32 bytes per lane and operand: 8 elements, or 16 when every tensor of a
  // chain is 16-bit (twice the bytes per interpreted step)
  bool wide = args.chain && region_is_16bit(args.out_type);
  for (int i = 0; i < args.ninputs; ++i) wide = wide && region_is_16bit(args.in[i].type);
  const int vec = wide ? 16 : 8;

  RegionGeometry g;
  const LaunchStatus planned = plan_fused_region(args, vec, block_dim, &g);
  if (planned.code != 0 || g.empty) return planned;
  const bool idx32 = g.idx32;
  if (args.reduce) {
    auto kernel = wide ? (idx32 ? fused_region_rowsum<int, true, 16> : fused_region_rowsum<int64_t, true, 16>)
                  : args.chain ? (idx32 ? fused_region_rowsum<int, true, 8> : fused_region_rowsum<int64_t, true, 8>)
                               : (idx32 ? fused_region_rowsum<int, false, 8> : fused_region_rowsum<int64_t, false, 8>);
    AFIR_LAUNCH("fused_region_rowsum", kernel, dim3((unsigned)g.blocks), dim3(kThreads), 0, stream, args, g.lanes_log2);
    return after_launch();
  }
  auto kernel = wide ? (idx32 ? fused_region_parallel<int, true, 16> : fused_region_parallel<int64_t, true, 16>)
                : args.chain ? (idx32 ? fused_region_parallel<int, true, 8> : fused_region_parallel<int64_t, true, 8>)
                             : (idx32 ? fused_region_parallel<int, false, 8> : fused_region_parallel<int64_t, false, 8>);
  AFIR_LAUNCH("fused_region_parallel", kernel, dim3((unsigned)(g.blocks / g.column_blocks), (unsigned)g.column_blocks), dim3(kThreads), 0,
                     stream, args, g.lanes_log2);
  return after_launch();
}

}  // namespace afir
