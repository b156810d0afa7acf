// Kernel-argument form of one segment of a fused-region program (see
// ../target/region_program.h for the program, region.hip for the kernel).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "common.h"

namespace afir {

constexpr int kRegionMaxInputs = 8;
constexpr int kRegionMaxOps = 32;
constexpr int kRegionMaxTail = 8;

enum RegionType : int { kRegionF16 = 0, kRegionBF16 = 1, kRegionF32 = 2, kRegionI32 = 3, kRegionI64 = 4, kRegionI16 = 5 };
// Values travel through float registers; an integer region keeps 32-bit two's
// complement integers in them bit for bit and uses the *I operations.
enum RegionOpCode : int {
  kRegionPush = 0, kRegionConst, kRegionAdd, kRegionSub, kRegionMul, kRegionDiv, kRegionMax,
  kRegionMin, kRegionRelu, kRegionLeaky, kRegionNeg, kRegionDup,
  kRegionCastF16, kRegionCastBF16,   // round to that type (nearest even) and widen again
  kRegionAddI = 16, kRegionSubI, kRegionMulI, kRegionMaxI, kRegionMinI, kRegionReluI, kRegionNegI,
  // comparisons of an i16 region look at the low 16 bits of their operands (add, sub, mul
  // and neg agree modulo 2^16 whatever the upper bits hold, and the store truncates)
  kRegionMaxI16, kRegionMinI16, kRegionReluI16
};
__host__ __device__ inline bool region_is_binary(int code) {
  return (code >= kRegionAdd && code <= kRegionMin) || (code >= kRegionAddI && code <= kRegionMinI) ||
         code == kRegionMaxI16 || code == kRegionMinI16;
}
__host__ __device__ inline bool region_is_unary(int code) {
  return code == kRegionRelu || code == kRegionLeaky || code == kRegionNeg || code == kRegionReluI ||
         code == kRegionNegI || code == kRegionReluI16 || code == kRegionCastF16 || code == kRegionCastBF16;
}
__host__ __device__ inline bool region_is_16bit(int type) {
  return type == kRegionF16 || type == kRegionBF16 || type == kRegionI16;
}

struct RegionInput {
  const void *base;    // device pointer of the tensor
  const void *index;   // device pointer of the index tensor (gather), else null
  int64_t stride[3];   // elements per step of each iteration dim
  int64_t offset;      // constant element offset
  int64_t gstride;     // elements per index step
  int64_t gextent;     // valid indices are [0, gextent)
  int type;            // RegionType of the tensor
  int gdim;            // iteration dim that indexes the index tensor, -1 = no gather
  int gtype;           // kRegionI32 / kRegionI64
  int vec;             // 128-bit loads along the innermost dim are aligned
  int gvec;            // ... also after adding any multiple of gstride
  int pad;
};

struct RegionOp {
  int code;
  int input;
  float constant;
  int depth;   // Dup: entries below the top
  int dst;     // stack slot the operation writes, filled in by the launcher:
               // push / const / dup write a new top, a binary operation
               // combines slot dst with slot dst + 1, a unary one works in place
  int pad[3];
};

// Linear form of a program, derived by the launcher where the expression is a
// chain: acc = u0(x0); acc = u_k(acc (op_k) x_k) for each step.  Reversed
// operands (x - acc, x / acc) have their own codes.
constexpr int kRegionMaxSteps = 8;
enum RegionChainCode : int { kChainRSub = 32, kChainRDiv = 33, kChainRSubI = 34 };
struct RegionUnary {
  int code[2];      // kRegionRelu / kRegionLeaky / kRegionNeg
  float alpha[2];
  int count;
  int pad;
};
struct RegionStep {
  int bop;          // RegionOpCode of a binary operation, or a RegionChainCode
  int input;        // operand: index into RegionArgs::in, or -1 for `constant`
  float constant;
  int pad;
  RegionUnary after;
};

struct RegionArgs {
  int64_t size[3];
  void *out;            // first element this segment writes
  int32_t *error_flag;  // set to 1 when a gathered index is out of range (may be null)
  int out_type;
  int out_vec;          // 128-bit stores are aligned for every full vector
  int rank;
  int nops;
  int ninputs;
  int reduce;
  RegionInput in[kRegionMaxInputs];
  RegionOp ops[kRegionMaxOps];
  // reduce segments: what happens to a row's sum s before it is stored, step by step:
  // s = s (code) constant, or constant (code) s with depth = 1, or a unary operation
  int ntail;
  int pad_tail;
  RegionOp tail[kRegionMaxTail];
  // filled in by the launcher
  int chain;              // 1: the fields below describe the whole expression
  int chain_first;        // x0: index into `in`, or -1 for chain_constant
  float chain_constant;
  int nsteps;
  RegionUnary chain_after_first;
  RegionStep steps[kRegionMaxSteps];
};

LaunchStatus launch_fused_region(const RegionArgs &args, uint32_t block_dim, hipStream_t stream);

// Launch geometry of a segment for `vec` elements per lane and step: shared by
// the interpreter kernels and by kernels compiled for one program.
struct RegionGeometry {
  int64_t blocks = 0;    // workgroups of 256 lanes (parallel segments: row blocks x column blocks)
  int64_t column_blocks = 1;   // parallel segments: workgroups that share a pass of rows, each taking
                               // every column_blocks-th stretch of 2^lanes_log2 lane-loads of the row
  int lanes_log2 = 0;    // parallel segments: 2^lanes_log2 lanes share a row
  bool idx32 = false;    // every position fits 32 bits
  bool empty = false;    // nothing to compute
};
LaunchStatus plan_fused_region(const RegionArgs &args, int vec, uint32_t block_dim, RegionGeometry *geometry);

}  // namespace afir
