// Fused-region programs: what a fused AFIR / linalg region becomes on this
// backend when it is not one of the hand-tuned kernel families.
//
// The reference lowers a fused region to generated AscendC source
// (lib/Conversion/LinalgToAscendC/ComputeConversion.cpp:246-750 reduction
// generics, :1290-1640 parallel generics with Identity / PureBroadcast /
// PureTranspose / BroadcastTranspose input maps and inlined addf / mulf /
// maximumf bodies, :828-1272 the fused gather row loop; concat of two chains
// in examples/add-broadcast-concat).  Here the same region is described by a
// small program that one generic gfx950 kernel executes: per output element a
// postfix expression over input reads, each read addressed through the affine
// map of the linalg operand (iteration dim, constant, or "index taken from an
// index tensor" for gathers), optionally followed by a row reduction.  The
// program plays the part of the device binary: it is registered with the
// kernel library, which hands back a handle to launch by (the shape of
// rtDevBinaryRegister / rtFunctionRegister + rtKernelLaunch,
// lib/Runtime/Execution/NativeExecutionRunner.cpp:332-369,476-488).
//
// Arithmetic is float32 with one round-to-nearest-even to the output type,
// like the reference's numpy goldens (examples/*/gen_data.py).  A region whose
// output is i16 or i32 is an integer region (afir.add / sub / mul / maximum /
// minimum / neg / relu on I16, I32: include/Dialect/AFIR/Ops/Basic/math.td:71-98):
// every read is i16 or i32, arithmetic is 32-bit two's complement (wrapping),
// the result is truncated to the output type; div, leaky relu, reductions and
// matmul are float-only.
//
// Text form (one item per line, '#' starts a comment):
//   afir-hip-region 1
//   arg in  <f16|bf16|f32|i16|i32|i64> <rank>      one line per function argument,
//   arg out <f16|bf16|f32|i16|i32> <rank>              inputs first, then the output
//   segment <iteration rank>
//     size <ref> <ref> ...      extent of each iteration dim: argA.D or a constant
//     outoff <ref> [<ref> ...]  first output row (dim 0) this segment writes: the sum of the terms
//     push argA <m0> <m1> ... [slice <ref> ...]
//                               read input A; m_r is d<k> (iteration dim k), an
//                               integer constant, or g<k>:argI (dim r is indexed
//                               by the rank-1 index tensor I at iteration dim k)
//                               slice: per-dim start offsets of an extract_slice
//     matmul argA argB [ta] [tb]
//                               push sum_k A[d0,k] * B[k,d1] (float32 accumulation); only as
//                               the first operation of a rank-2 segment.  ta: A is stored
//                               transposed, [K,M]; tb: B is stored as [N,K]
//                               (linalg.matmul_transpose_a / _b).  Opening a rank-3 segment
//                               it is the batched product out[b] = A[b] x B[b] of rank-3
//                               operands (linalg.batch_matmul*), d0 being the batch
//     const <float>             push a constant
//     const <ref> [<type>]      push an extent as a number (mean = sum / N): the value of
//                               argA.D converted to float, rounded to f16 | bf16 when a
//                               type is given (arith.sitofp of a tensor.dim to that type)
//     add | sub | mul | div | max | min      pop b, pop a, push a op b
//     relu | leaky <alpha> | neg             on the top of the stack
//     cast <f16|bf16|f32>       round the top of the stack to that type and widen it again
//                               (arith.truncf / arith.extf, afir.cast; a row sum that the IR
//                               keeps in a narrower tensor before the next operation reads it)
//     dup <n>                   push a copy of the n-th entry from the top
//     reduce sum                sum the value over the last iteration dim
//     ...                       after 'reduce sum': operations on the row's sum with constants
//                               and extents only (const, the binary and unary operations,
//                               dup; no push), e.g. 'const arg1.1 f16' 'div' for a mean
//     store                     round to the output type and write
//   end
#pragma once

#include <cstdint>
#include <string>
#include <vector>

namespace afir_region {

enum class ElemType { F16, BF16, F32, I32, I64, I16 };
const char *elemTypeName(ElemType t);
size_t elemTypeBytes(ElemType t);
bool parseElemType(const std::string &s, ElemType *out);
inline bool isFloat(ElemType t) { return t == ElemType::F16 || t == ElemType::BF16 || t == ElemType::F32; }
// Element types of integer regions (i64 serves as an index type only).
inline bool isRegionInt(ElemType t) { return t == ElemType::I16 || t == ElemType::I32; }

constexpr int kMaxRank = 3;       // iteration rank and tensor rank
constexpr int kMaxArgs = 10;      // inputs + output
constexpr int kMaxOps = 32;
constexpr int kMaxStack = 4;

struct Arg {
  bool isOutput = false;
  ElemType type = ElemType::F32;
  int rank = 0;
};

// An extent or offset: a dimension of an argument, or a constant.
struct Ref {
  int arg = -1;  // -1: constant
  int dim = 0;
  int64_t constant = 0;
  static Ref dimOf(int a, int d) { Ref r; r.arg = a; r.dim = d; return r; }
  static Ref value(int64_t c) { Ref r; r.constant = c; return r; }
};

enum class OpCode { Push, Const, Add, Sub, Mul, Div, Max, Min, Relu, Leaky, Neg, Dup, ReduceSum, Store, Matmul, Cast };

struct MapResult {
  enum Kind { IterDim, Constant, Gather } kind = IterDim;
  int iterDim = 0;       // IterDim: which; Gather: iteration dim that indexes the index tensor
  int64_t constant = 0;  // Constant
  int indexArg = -1;     // Gather: the rank-1 index tensor
};

struct Op {
  OpCode code = OpCode::Add;
  int arg = -1;                     // Push; Matmul: the [M,K] operand
  int arg2 = -1;                    // Matmul: the [K,N] operand
  bool transA = false, transB = false;   // Matmul: the operand is stored transposed
  std::vector<MapResult> map;       // Push: one per dim of the input
  std::vector<Ref> slice;           // Push: start offset per dim (empty = none)
  float constant = 0.f;             // Const, Leaky
  bool extent = false;              // Const: the value is an extent (constRef), not `constant`
  Ref constRef;                     // Const with extent set
  ElemType constType = ElemType::F32;  // ... rounded through this float type; Cast: the type
  int depth = 0;                    // Dup
};

struct Segment {
  int rank = 0;
  std::vector<Ref> sizes;
  Ref outOffset = Ref::value(0);
  std::vector<Ref> outOffsetMore;   // further terms added to outOffset (concat of 3+ dynamic parts)
  std::vector<Op> ops;
  bool reduces() const;
};

struct Program {
  std::vector<Arg> args;           // inputs..., output (exactly one output, last)
  std::vector<Segment> segments;
  int numInputs() const { return (int)args.size() - 1; }
  const Arg &output() const { return args.back(); }
};

std::string serialize(const Program &p);
// Empty string on success, else the diagnostic.
std::string parse(const std::string &text, Program *out);
// Structural checks: stack discipline, ranks, references, one store per
// segment at the end, gathers index with integer rank-1 tensors, ...
std::string validate(const Program &p);

// TilingData of a program: one int64 per dimension of every argument,
// dim_arg<A>_<D> in argument order (the naming of the reference's generated
// TilingData, lib/Conversion/AscendCPrepareForEmit/AscendCPrepareForEmitPass.cpp:107-254).
std::vector<std::string> tilingFieldNames(const Program &p);

// ---- resolution against concrete shapes ------------------------------------

struct ResolvedInput {
  int arg = 0;
  ElemType type = ElemType::F32;
  int64_t iterStride[kMaxRank] = {0, 0, 0};  // elements per step of each iteration dim
  int64_t offset = 0;                        // constant element offset (constants, slices)
  int gatherIterDim = -1;                    // >= 0: dim indexed through an index tensor
  int gatherIndexArg = -1;
  ElemType gatherIndexType = ElemType::I64;
  int64_t gatherStride = 0;                  // elements per index step
  int64_t gatherExtent = 0;                  // valid indices are [0, extent)
};

struct ResolvedOp {
  OpCode code = OpCode::Add;
  int input = -1;      // Push: index into ResolvedSegment::inputs
  int arg = -1, arg2 = -1;  // Matmul: argument indices
  int64_t k = 0;            // Matmul: contraction extent
  int64_t batch = 1;        // Matmul: independent products (rank-3 segment)
  bool transA = false, transB = false;
  float constant = 0.f;
  int depth = 0;
  ElemType castType = ElemType::F32;   // Cast
};

struct ResolvedSegment {
  int rank = 0;
  int64_t size[kMaxRank] = {1, 1, 1};
  bool reduce = false;
  int64_t outOffsetElems = 0;   // element offset of this segment's first output element
  int64_t outElems = 0;         // elements this segment writes
  ElemType outType = ElemType::F32;
  std::vector<ResolvedInput> inputs;
  std::vector<ResolvedOp> ops;    // up to and including 'reduce sum' (all of them without one), and 'store'
  // What follows 'reduce sum', as a chain on the row's sum s (operations among constants are
  // folded, in float32): s = s op c, or c op s when reversed (sub, div), or a unary operation.
  struct TailStep {
    OpCode code = OpCode::Add;
    float constant = 0.f;   // the other operand; alpha of Leaky
    bool reversed = false;
    ElemType castType = ElemType::F32;   // Cast
  };
  std::vector<TailStep> tail;
};

constexpr int kMaxTailOps = 8;    // operations on the sum between 'reduce sum' and 'store'
constexpr int kMaxTailExtents = 4;   // of which extent constants
constexpr int kMaxSegmentExtents = 8;   // extent constants of one segment, before and after 'reduce sum'

// float -> f16 / bf16 -> float, round to nearest even (f32: the value itself).
float roundThroughType(float f, ElemType t);

struct Resolved {
  std::vector<std::vector<int64_t>> shapes;  // per argument
  std::vector<size_t> bytes;                 // per argument
  std::vector<ResolvedSegment> segments;
};

// dims: the TilingData values in tilingFieldNames order.  Checks that every
// read stays inside its tensor, that segment sizes agree with the shapes they
// refer to and that the segments tile the output exactly.
std::string resolve(const Program &p, const std::vector<int64_t> &dims, Resolved *out);

}  // namespace afir_region
