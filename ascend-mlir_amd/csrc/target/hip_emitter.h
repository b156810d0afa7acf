// Fused-region program -> HIP source of a kernel specialised for it: what the
// reference's emitter does for AscendC (lib/Target/CannKernel/CannTranslation.cpp:2487-2694
// prints one C++ kernel per fused region; the compute bodies come from
// lib/Conversion/LinalgToAscendC/ComputeConversion.cpp:1290-1640 for parallel
// generics, :246-750 for reductions, :828-1272 for the fused gather loop).
//
// The emitted source needs no headers (it uses compiler builtins only), so
// compiling it to a code object takes a fraction of a second:
//   hipcc --genco --offload-arch=gfx950 -O3 -nogpuinc -ffp-contract=off
//         -Xclang -target-feature -Xclang -packed-fp32-ops -o region.hsaco region.hip
// The code object is attached to the registered program
// (afir_hip_region_attach_code_object) and launched in place of the generic
// interpreter kernel; parallel segments give the same bits as that kernel, row
// sums (float32 sums in another, fixed order) agree within rounding.
//
// What is fixed at emission: the iteration rank, the operation sequence, the
// element types, which operands are broadcast / contiguous / strided / gathered
// along the innermost dim.  What stays a launch argument: pointers, extents,
// strides, offsets, alignment of this particular launch.
#pragma once

#include <cstdint>
#include <string>
#include <vector>

#include "region_program.h"

namespace afir_target {

// Launch argument of every emitted kernel.  The emitted source carries the same
// declaration and static_asserts its size and field offsets against this one.
struct SpecInput {
  const void *base;    // device pointer of the tensor
  const void *index;   // device pointer of the index tensor (gather), else null
  long long stride[3]; // elements per step of each iteration dim
  long long offset;    // constant element offset
  long long gstride;   // elements per index step
  long long gextent;   // valid indices are [0, gextent)
  int vec;             // 128-bit loads along the innermost dim are aligned
  int gvec;            // ... also after adding any multiple of gstride
};
constexpr int kSpecMaxInputs = 8;
constexpr int kSpecMaxExtentConsts = afir_region::kMaxSegmentExtents;
struct SpecArgs {
  long long size[3];
  void *out;
  int *error_flag;     // set to 1 when a gathered index is out of range (may be null)
  int out_vec;         // 128-bit stores are aligned for every full vector
  int lanes_log2;      // parallel segments: lanes of the workgroup that share a row
  int grid;            // number of workgroups launched
  int column_blocks;   // parallel segments: of these, the workgroups that share a pass of rows and
                       // split the row between them (grid is a multiple of it; 1 elsewhere)
  SpecInput in[kSpecMaxInputs];
  float extent_const[kSpecMaxExtentConsts];   // the segment's extent constants ('const argA.D'), in program
                                              // order, before and after 'reduce sum' (resolved per launch)
  int hold_ticks;      // phased kernels: ticks of the real-time counter a workgroup holds its stores back
  int first_block;     // phased kernels: number of the launch's first workgroup (a shape sent as two launches)
};
// The values of a segment's extent constants for a launch's shapes (what goes into
// SpecArgs::extent_const): shapes[a][d] = extent of dim d of argument a.
void specExtentConstants(const afir_region::Program &p, int segment,
                         const std::vector<std::vector<int64_t>> &shapes, float (&out)[kSpecMaxExtentConsts]);

// Programs of 2..kSpecMaxSegments segments also get one kernel that runs all
// of them in a single launch (segments write disjoint row ranges of the
// output); its argument:
constexpr int kSpecMaxSegments = 4;
struct SpecAll {
  int first[kSpecMaxSegments + 1];   // first workgroup of each segment, then the total
  int pad;
  SpecArgs seg[kSpecMaxSegments];    // the emitted declaration holds the program's segment count
};
std::string specAllKernelName(bool idx32, int mode);
bool specAllSegments(const afir_region::Program &p);   // whether that kernel is emitted

// A parallel segment that reads an operand transposed (contiguous along an
// outer iteration dim `dim`, strided along the innermost one) is walked in
// tiles of EmitOptions::tileP (dim) x tileQ (innermost dim), the transposed
// operands staged through LDS; the launch then has one workgroup pass per tile.
struct SpecTile {
  bool tiled = false;
  int dim = -1;
  unsigned inputs = 0;   // bit i: SpecArgs::in[i] is staged through LDS; its `vec` flag then
                         // means "128-bit loads along `dim` are aligned"
};
SpecTile specTile(const afir_region::Program &p, int segment);

// Choices the emitter leaves open: the tile of segments that read an operand
// transposed, and how many groups a lane takes per pass elsewhere.  They are
// compile-time constants of the emitted kernels; the code object exports them
// (`afir_region_emit_options`) so that the launcher sizes its grids to match.
struct EmitOptions {
  int tileP = 64;   // tile extent along the dim the transposed operands are contiguous in (multiple of 32)
  int tileQ = 64;   // tile extent along the innermost iteration dim (64, 128 or 256)
  int unroll = 0;   // groups per lane and pass in untiled segments; 0 = by element types (4, or 2 when mixed)
};
// "" if usable, else why not.
std::string checkEmitOptions(const EmitOptions &o);
// "tile_p" / "tile_q" / "unroll" = integer; returns false for an unknown name.
bool setEmitOption(EmitOptions *o, const std::string &name, long long value);

// A lane's share of one pass over a row: `unroll` groups of `width` consecutive
// elements (16 bytes of the narrowest tensor), the groups one lane-set apart.
struct SpecShape {
  int width = 8;
  int unroll = 2;
};
SpecShape specShape(const afir_region::Program &p, int segment, const EmitOptions &options = EmitOptions());

// FNV-1a of the serialized program: the emitted code object exports it as
// `afir_region_program_hash`, checked when the code object is attached.
uint64_t programHash(const afir_region::Program &p);

// Version of the set of kernels and of the launch arguments that emitHipSource produces; the
// code object exports it as `afir_region_emit_abi`, and a code object of another version is
// refused when it is loaded (its kernels would be launched with the wrong names or arguments).
constexpr int kSpecAbiVersion = 10;

// What a launch promises, which picks the kernel variant:
//   kSpecAligned  every 128-bit access is aligned and every pass of the lanes over a row is whole
//   kSpecVector   every 128-bit access is aligned and the innermost extent is a multiple of the
//                 lane width; the last pass may be partly empty (not emitted for tiled segments)
//   kSpecGeneral  anything: tails and unaligned tensors take element accesses
enum SpecMode { kSpecGeneral = 0, kSpecVector = 1, kSpecAligned = 2 };
// Kernel symbol of a segment: idx32 = positions fit 32 bits.
std::string specKernelName(int segment, bool idx32, int mode);
// Untiled segments also have kernels whose lanes take one group each, for rows of
// fewer than 8 x unroll groups (32-bit positions, modes kSpecAligned and kSpecVector).
std::string specSlimKernelName(int segment, int mode);
// A parallel rank-2 segment with one operand gathered along the innermost dim from the rows
// of a matrix (`x[d0, index[d1]]`, the reference example's column gather) also has kernels
// that stage the operand's source row in LDS, a workgroup per row, and gather from there:
// launched with gextent * elemBytes bytes of dynamic LDS when the source rows are contiguous,
// 16-byte aligned, a whole number of 128-bit chunks and at most kSpecStageBytes long.
struct SpecStage {
  int input = -1;      // SpecArgs::in slot of that operand, -1: the segment has no such kernels
  int elemBytes = 2;
};
SpecStage specStage(const afir_region::Program &p, int segment);
constexpr int kSpecStageBytes = 64 * 1024;
// wave: the variant that gives a wavefront to a row (four rows per workgroup, each with its own
// gextent * elemBytes bytes of the LDS, no barriers), for output rows of at most two passes of
// a wavefront.
std::string specStagedKernelName(int segment, bool idx32, int mode, bool wave);
// ... and kernels whose groups are single elements (kSpecElementUnroll of them per lane, a
// lane-set apart), launched when rows do not start on 16-byte boundaries: every load and
// store instruction of a wavefront then still covers one contiguous run.
constexpr int kSpecElementUnroll = 8;
std::string specElementKernelName(int segment, bool idx32);
// Reduce segments also have a workgroup-per-row kernel for rows of exactly
// 256 * unroll * width elements whose accesses are all 128-bit.
std::string specRowsKernelName(int segment, bool idx32);
// ... and one for rows of a whole number (two or more) of such stretches, launched when the
// rows are too few to fill the chip with a wavefront each.
std::string specLongRowsKernelName(int segment, bool idx32);
// ... and a pair for a handful of such rows: `split` (column_blocks workgroups per row, each
// leaving a partial sum in the code object's afir_region_partials) and `join` (a wavefront per
// row adds them in a fixed order).  rows x column_blocks may not exceed kSpecPartials.
constexpr int kSpecPartials = 65536;
std::string specSplitRowsKernelName(int segment, bool idx32, bool join);

// A parallel segment whose operands are of three kinds only -- streamed (contiguous along the
// innermost dim and addressed by every outer dim, or rows gathered through an index tensor along
// an outer dim: one or two of them), row vectors (contiguous along the innermost dim, the same for
// every row: up to four) and values broadcast along the innermost dim -- with every streamed
// operand, row vector and the output of one element size, also has a kernel that separates its
// reads from its writes in time: every lane of the launch is resident at once, takes
// kSpecPhasedGroups groups of 16 bytes of output, computes them as its loads arrive (in as many
// rounds as there are streamed operands), keeps the packed results in registers and stores them
// once SpecArgs::hold_ticks of the real-time counter have passed since the workgroup started.
// Launched with 32-bit positions for shapes of whole workgroups whose accesses are all aligned:
// rows of 8 * 2^k groups, k <= 8, a workgroup covering 256 >> k rows (lanes_log2 = k,
// column_blocks = 1; the row vectors staged in `vectors x row bytes` of dynamic LDS), or rows of a
// multiple of 2048 groups without row vectors (lanes_log2 = 8, column_blocks = stretches per row).
struct SpecPhased {
  bool eligible = false;
  int streamed = 0;      // operands read once per output element: the rounds of the kernel
  int vectors = 0;       // row vectors staged in LDS
  int elemBytes = 4;     // element size of the output, the streamed operands and the row vectors
};
constexpr int kSpecPhasedGroups = 8;
constexpr int kSpecPhasedMaxVectors = 4;
SpecPhased specPhased(const afir_region::Program &p, int segment);
std::string specPhasedKernelName(int segment);
std::string specAllPhasedKernelName();   // every segment of a program in one such launch

// Emits the source for every segment.  Returns "" on success, else why the
// program has no specialised form (matmul segments: those run on the
// hand-written kernels).
std::string emitHipSource(const afir_region::Program &p, const std::string &title, std::string *source,
                          const EmitOptions &options = EmitOptions());

// The compiler invocation for a source file (argv, no shell).
std::string hipccCommandLine(const std::string &sourcePath, const std::string &outputPath);

}  // namespace afir_target
