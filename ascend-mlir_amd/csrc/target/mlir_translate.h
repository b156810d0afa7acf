// MLIR text -> fused-region program: the HIP sibling of the reference's
// `afir-translate -mlir-to-cann` (tools/afir-translate/afir-translate.cpp:19-41,
// lib/Target/CannKernel/CannTranslation.cpp:2487-2694).
//
// The reference reaches its emitter through a pipeline of MLIR passes
// (--linalg-fuse-elementwise-ops, --mark-structured-ops,
// --fuse-gather-elementwise, --linalg-to-ascendc ...,
// examples/broadcast-add-reduce/run.sh:52-200).  There is no MLIR library to
// link here, so this reads the textual IR of the supported subset directly and
// does the part of those passes that decides WHAT the kernel computes:
//
//   - linalg.generic with parallel iterators: the body (arith.addf / subf /
//     mulf / divf / maximumf / minimumf / negf, constants) is inlined into its
//     consumers through the operands' affine maps, which is what
//     --linalg-fuse-elementwise-ops does for the three generics of an example;
//     map classes as in lib/Conversion/LinalgToAscendC/ComputeConversion.cpp:265-333
//     (identity, broadcast, transposed, constant results);
//   - tensor.extract inside a generic with one index taken from an index
//     tensor: the gather of lib/Conversion/MarkStructuredOps/MarkStructuredOpsPass.cpp:54-147,
//     fused with its producer and consumer as
//     lib/Conversion/FuseGatherElementwise/FuseGatherElementwisePass.cpp:61-303 does;
//   - a generic whose last iterator is a reduction with an addf accumulation
//     over a zero-filled init: the row sum of ComputeConversion.cpp:428-750;
//   - linalg.matmul followed by a bias add and max(x, x*alpha): the
//     BiasAddLeakyRelu epilogue of
//     lib/Conversion/MarkStructuredOps/AnnotateMixMatmulSemanticsPass.cpp:79-342;
//   - tensor.extract_slice / tensor.concat along dim 0
//     (examples/split-relu-brc-add-mul, examples/add-broadcast-concat);
//   - AFIR ops in their custom syntax (afir.add / sub / mul / div / maximum /
//     minimum with numpy-style broadcasting, relu, leaky_relu{negative_slop},
//     neg, broadcast, sum{axis = last}, load / store as the identity; include/Dialect/AFIR/Ops/Basic/math.td:63-106,
//     lib/Dialect/AFIR/Ops/Basic/math.cpp:274-381).
// Anything else is rejected with a diagnostic naming the construct.
#pragma once

#include <string>

#include "region_program.h"

namespace afir_target {

struct Translation {
  std::string functionName;
  afir_region::Program program;
};

// For files that hold several functions (the reference's lit tests do): the
// text with everything between the leading aliases / module header and
// `func.func @name` removed, so that it is the first function.  Returns "" when
// there is no such function.
std::string selectFunction(const std::string &mlirText, const std::string &name);

// Translates the first func.func of `mlirText`.  Returns "" on success, else
// the diagnostic ("line N: ...").
std::string translateMlirToRegion(const std::string &mlirText, Translation *out);

// {"tiling_params": [{"name": "dim_arg0_0", "type": "int64"}, ...]} -- the
// skeleton the reference's --tiling-space-out writes
// (lib/Target/CannKernel/CannTranslation.cpp:1987-2042), with this backend's
// fields.
std::string tilingSpaceJson(const afir_region::Program &program, const std::string &kernelName);

}  // namespace afir_target
