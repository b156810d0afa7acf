/*
 * afir_hip_kernels.h — C ABI of the gfx950 fused-kernel library
 * (libafir_hip_kernels.so).
 *
 * This is the seam the reference runtime already has for "a shared library
 * that exports one launcher symbol per kernel": its runner dlopen()s the
 * artifact, dlsym()s the symbol and calls
 *
 *     uint32_t fn(uint32_t blockDim, void *stream, void *a0 ... void *a15)
 *
 * with [inputs..., outputs..., workspace, tiling], non-zero meaning failure,
 * and synchronises the stream afterwards
 * (reference: lib/Runtime/Execution/NativeExecutionRunner.cpp:616-636,753-785;
 * generated launcher prototype lib/Runtime/Mix/MixStubTemplate.cpp:57-77).
 * Every launcher below has exactly that shape, so a runner that binds the
 * reference's dynamic-library artifacts binds these without a new call path.
 *
 * Conventions
 *   - all tensor pointers are DEVICE pointers, row-major, densely packed;
 *   - `stream` is a hipStream_t (NULL = the default stream); launches are
 *     asynchronous, the caller synchronises;
 *   - `tiling` points to HOST memory holding the packed TilingData of the
 *     kernel: little-endian int64 fields in the order documented per kernel
 *     (the byte string the reference's TilingSchema::pack produces,
 *     lib/Runtime/Support/TilingSchema.cpp:61-100).  HIP passes kernel
 *     arguments by value, so the launcher reads the shapes on the host — the
 *     reference's vec-kernel convention of passing tiling as trailing words of
 *     the argument buffer (NativeExecutionRunner.cpp:438-454) rather than its
 *     mix-kernel convention of a device copy;
 *   - field names follow the reference's generated TilingData:
 *     dim_arg<A>_<D> = extent of dimension D of argument A, arguments counted
 *     over (inputs..., outputs...)
 *     (lib/Conversion/AscendCPrepareForEmit/AscendCPrepareForEmitPass.cpp:107-254);
 *   - `block_dim` = number of workgroups to launch; 0 lets the launcher size
 *     the grid for the 256 CUs of an MI355X (every kernel is grid-strided, so
 *     any positive value is correct);
 *   - `workspace` may be NULL unless stated; kernels that report data errors
 *     (gather index out of range) set the first 4 bytes to non-zero when it is
 *     given;
 *   - return 0 on success, AFIR_HIP_E_* otherwise; afir_hip_last_error()
 *     returns the calling thread's last message.
 *
 * Numerics: every kernel computes in float32 and rounds once (nearest even)
 * to the storage type, like the reference's numpy goldens
 * (examples/xx/gen_data.py: "compute in f32, cast to storage dtype").
 */
#ifndef AFIR_HIP_KERNELS_H
#define AFIR_HIP_KERNELS_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define AFIR_HIP_OK 0u
#define AFIR_HIP_E_INVALID 1u  /* bad pointer / shape / tiling bytes          */
#define AFIR_HIP_E_LAUNCH 2u   /* HIP reported an error at launch             */
#define AFIR_HIP_E_UNKNOWN 3u  /* no kernel of that name                      */

/* Message for the calling thread's most recent non-zero return ("" if none). */
const char *afir_hip_last_error(void);

/* The kernel the calling thread launched last through this library: its name
 * (a static or thread-owned string, "" before the first launch), the number of
 * workgroups and the lanes per workgroup.  A launcher call may launch several
 * kernels (two halves of a large shape, split + join); this is the last one.
 * Either pointer may be NULL.  No counterpart in the reference, whose launches
 * take the caller's block_dim as given; here block_dim 0 leaves the grid to
 * the launcher and a runner reports what it chose. */
const char *afir_hip_last_launch(uint32_t *workgroups, uint32_t *threads);

/* ---- fused elementwise chain: out = (a + b) * b ---------------------------
 * Replaces the lowering of afir.add -> afir.mul
 * (lib/Conversion/AFIRToASCIR/Math/Elementwise.cpp:25-57; chain from
 * README.md:191-197).  f32, a/b/out of identical shape.
 * TilingData { int64 dim_arg0_0 (rows); int64 dim_arg0_1 (cols); }            */
uint32_t afir_hip_launch_fused_add_mul(uint32_t block_dim, void *stream,
                                       void *a, void *b, void *out,
                                       void *workspace, void *tiling);

/* ---- broadcast add + row sum: y[i] = sum_j (x[i,j] + bias[j]) -------------
 * Replaces the reduction-generic lowering
 * (lib/Conversion/LinalgToAscendC/ComputeConversion.cpp:246-750, emitted
 * ReduceSum at lib/Target/CannKernel/CannTranslation.cpp:2384-2484).
 * f32 x[M,N], bias[N], y[M]; float32 accumulation.
 * TilingData { int64 dim_arg0_0 (M); int64 dim_arg0_1 (N); }                  */
uint32_t afir_hip_launch_broadcast_add_reducesum(uint32_t block_dim, void *stream,
                                                 void *x, void *bias, void *y,
                                                 void *workspace, void *tiling);

/* The same computation for callers that must not allocate (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc).  No
 * counterpart in the reference.  The launcher above may load a code object on
 * first use and its split-and-join form for few, long rows keeps partial sums
 * in that code object; this one calls no hipMalloc, hipFree or other
 * allocating routine.  Rows are split when M < 1024 and N >= 16384 (chunks of
 * 8192 floats, one partial sum each, added in a fixed order by a second
 * kernel); the partial sums live in a 256 KiB array that the library holds on
 * every GPU it runs on until the process ends, so M * ceil(N / 8192) must not
 * exceed 65536: beyond that the call returns AFIR_HIP_E_NOALLOC_LIMIT and
 * launches nothing.  Other shapes run the scratch-free kernels of the launcher
 * above.  `workspace` is ignored.  Every call on a GPU shares that GPU's array
 * (nothing in it has to start at zero: each partial sum is written before it
 * is read), so calls that overlap on one GPU -- other streams, other threads
 * -- race; serialise them.  Returns the code only: afir_hip_last_error() is
 * not updated. */
#define AFIR_HIP_E_NOALLOC_LIMIT 4u
uint32_t afir_hip_launch_broadcast_add_reducesum_noalloc(uint32_t block_dim, void *stream,
                                                         void *x, void *bias, void *y,
                                                         void *workspace, void *tiling);

/* ---- relu + broadcast add + transpose ------------------------------------
 * out[b,j,i] = f16(relu(x[b,i,j]) + c[j]); x f16 [B,M,N], c f16 [N],
 * out f16 [B,N,M].  Replaces the parallel generic with a PureTranspose input
 * map and a PureBroadcast input (ComputeConversion.cpp:265-333,1290-1640;
 * transpose emission :775-826).
 * TilingData { int64 dim_arg0_0 (B); int64 dim_arg0_1 (M); int64 dim_arg0_2 (N); } */
uint32_t afir_hip_launch_relu_broadcast_add_transpose(uint32_t block_dim, void *stream,
                                                      void *x, void *c, void *out,
                                                      void *workspace, void *tiling);

/* ---- row gather + scale + shift -------------------------------------------
 * out[r,:] = f16(table[indices[r],:] * scale + shift); table f16 [V,D],
 * indices int32 [R] in [0,V), scale/shift f16 [D], out f16 [R,D].
 * Replaces the fused gather region (--fuse-gather-elementwise,
 * lib/Conversion/FuseGatherElementwise/FuseGatherElementwisePass.cpp:61-303;
 * row loop ComputeConversion.cpp:828-1272) in its embedding (row) flavour
 * (lib/Conversion/MarkStructuredOps/MarkStructuredOpsPass.cpp:141-145).
 * An index outside [0,V) yields a row of NaN and, when workspace is given,
 * a non-zero int32 at workspace[0]; it never reads outside the table.
 * TilingData { int64 dim_arg0_0 (V); int64 dim_arg0_1 (D); int64 dim_arg1_0 (R); } */
uint32_t afir_hip_launch_gather_scale_shift(uint32_t block_dim, void *stream,
                                            void *table, void *indices,
                                            void *scale, void *shift, void *out,
                                            void *workspace, void *tiling);

/* ---- matmul + bias + leaky relu --------------------------------------------
 * out = bf16(leakyrelu(A @ B + bias, alpha)); A bf16 [M,K], B bf16 [K,N]
 * (not transposed), bias bf16 [N], out bf16 [M,N]; float32 accumulation on
 * the matrix cores, epilogue fused before the store.  leakyrelu(x) is
 * max(x, x*alpha) as the reference IR spells it
 * (examples/matmul-add-leakyrelu/step0_input.mlir:40-52).  Replaces the mix
 * kernel (lib/Target/CannKernel/CannTranslation.cpp:1573-1628,1848-1869;
 * epilogue vocabulary BiasAddLeakyRelu,
 * lib/Conversion/MarkStructuredOps/AnnotateMixMatmulSemanticsPass.cpp:79-342).
 * TilingData { int64 dim_arg0_0 (M); int64 dim_arg0_1 (K); int64 dim_arg1_1 (N);
 *              int64 alpha_f32_bits (IEEE-754 bits of alpha in the low 32 bits) } */
uint32_t afir_hip_launch_matmul_add_leakyrelu(uint32_t block_dim, void *stream,
                                              void *a, void *b, void *bias, void *out,
                                              void *workspace, void *tiling);

/* ---- registry + name-based dispatch -----------------------------------------
 * What a runner needs to bind a kernel by the name an artifact manifest
 * carries (kernel_name=..., lib/Runtime/Artifact/VecCubeArtifactBackend.cpp:62-106)
 * and to build its tiling schema. */
typedef struct AfirHipKernelInfo {
  const char *name;           /* e.g. "broadcast_add_reducesum"                */
  const char *symbol;         /* launcher symbol exported by this library       */
  int num_inputs;
  int num_outputs;
  int num_tiling_fields;
  const char *const *tiling_fields; /* names, in TilingData order, all int64   */
  const char *signature;      /* human-readable: dtypes and shapes             */
} AfirHipKernelInfo;

int afir_hip_kernel_count(void);
/* The family as a region program (text), or NULL when it has none (the matmul and the
 * plain add-mul chain).  The library's build compiles these programs to
 * lib/families/<family>.hsaco; a family launcher whose specialised kernels do not fit the
 * shapes of a launch (rows that are no multiple of the tile, short rows, few rows) runs it
 * on those kernels.  AFIR_HIP_FAMILY_FALLBACK=0 keeps every launch on the family's own
 * kernels.  No counterpart in the reference: its kernels are generated per graph. */
const char *afir_hip_family_program(const char *family);
const AfirHipKernelInfo *afir_hip_kernel_info(int index);
const AfirHipKernelInfo *afir_hip_find_kernel(const char *name);

/* Byte sizes of the tensor arguments [inputs..., outputs...] that a tiling
 * implies, so that a runner can check the caller's buffers on the host before
 * it launches (the C API above it carries byte counts but no shapes,
 * lib/CAPI/Runtime/Runtime.cpp:122-134).  Writes num_inputs + num_outputs
 * entries; max_args is the capacity of `bytes`. */
uint32_t afir_hip_argument_bytes(const char *kernel_name, const void *tiling, size_t tiling_len,
                                 size_t *bytes, int max_args);

/* Launch by name.  args = [inputs..., outputs...] device pointers
 * (num_args must equal num_inputs + num_outputs of the kernel); tiling_len is
 * checked against 8 * num_tiling_fields. */
uint32_t afir_hip_launch(const char *kernel_name, uint32_t block_dim, void *stream,
                         int num_args, void *const *args, void *workspace,
                         const void *tiling, size_t tiling_len);

/* ---- fused-region programs -----------------------------------------------------
 * A fused region that is none of the families above (any chain of
 * add/sub/mul/div/max/min/relu/leaky_relu over inputs read through broadcast,
 * transposed, constant or gathered index maps, optionally summed over the last
 * dim, optionally concatenated along dim 0) runs on one generic kernel that
 * executes a region PROGRAM -- the text a translator derives from the region's
 * IR (grammar: csrc/target/region_program.h).  The program stands where the
 * reference has a device binary: it is registered once and launched by handle,
 * the shape of rtDevBinaryRegister / rtFunctionRegister followed by
 * rtKernelLaunch(handle, block_dim, args...)
 * (lib/Runtime/Execution/NativeExecutionRunner.cpp:332-369,476-488).
 *
 * TilingData of a program: one int64 per dimension of every argument,
 * dim_arg<A>_<D>, arguments in declaration order (inputs..., output);
 * afir_hip_region_tiling_field names them.  args = device pointers in the same
 * order.  workspace as for the launchers (int32 error flag for gathers). */
uint32_t afir_hip_region_register(const char *program_text, size_t program_len, uint64_t *handle);
uint32_t afir_hip_region_unregister(uint64_t handle);
uint32_t afir_hip_region_info(uint64_t handle, int *num_inputs, int *num_outputs,
                              int *num_tiling_fields);
/* Which kernel runs the program: one of the family names above when the
 * program is exactly that family (it is then routed to the hand-tuned kernel),
 * else "fused_region" (the generic kernel).  Setting the environment variable
 * AFIR_HIP_REGION_GENERIC=1 before registering keeps every non-matmul program
 * on the generic kernel. */
const char *afir_hip_region_kernel(uint64_t handle);
/* Which of the three routes a launch with these shapes takes (tiling as for
 * afir_hip_launch_region; host only, launches nothing):
 *   "family"       the hand-tuned kernel afir_hip_region_kernel names.  Those
 *                  kernels take densely packed operands of exactly the
 *                  iteration extents, so a program of a family's form whose
 *                  launch reads part of a larger tensor (a zero-offset slice
 *                  narrower than its operand) does not take it;
 *   "compiled"     the kernels of the attached code object;
 *   "interpreter"  the library's interpreter kernel: correct for every
 *                  program, at a fraction of the compiled kernels' rate.
 * "" with afir_hip_last_error() set when the shapes do not resolve.  The
 * reference announces how a task was run in its session.runtime.attribute.*
 * lines (tools/runtime-session/runtime_session_main.cpp:161-183); this is the
 * source of the region_route attribute there. */
const char *afir_hip_region_route(uint64_t handle, const void *tiling, size_t tiling_len);
/* Kernels compiled for one program, the counterpart of the reference's
 * generated kernel source and device binary
 * (lib/Target/CannKernel/CannTranslation.cpp:2487-2694 prints the source,
 * lib/Runtime/Execution/NativeExecutionRunner.cpp:332-369 registers the
 * binary).  emit_source writes the HIP source for the program (NUL-terminated,
 * truncated to `capacity`; *length = full length, so call with a null buffer
 * first).  It is compiled with
 *   hipcc --genco --offload-arch=gfx950 -O3 -nogpuinc -ffp-contract=off
 *         -Xclang -target-feature -Xclang -packed-fp32-ops -o region.hsaco region.hip
 * and the resulting file's bytes are handed to attach_code_object; the launches
 * of that handle then run the compiled kernels ("fused_region_compiled")
 * instead of the interpreter, with bit-identical results.  The image is checked
 * against the program when it is first launched (AFIR_HIP_E_LAUNCH if it was
 * built from another program).  Programs routed to a hand-tuned family keep
 * that kernel.  Matmul programs have no source form (AFIR_HIP_E_INVALID). */
uint32_t afir_hip_region_emit_source(uint64_t handle, char *buffer, size_t capacity, size_t *length);
uint32_t afir_hip_region_attach_code_object(uint64_t handle, const void *image, size_t image_len);
/* Loads the attached code object on the current device now and checks it against
 * the program (hash, kernel-set version), which the first launch would otherwise
 * do: for callers that time their first launch or are about to capture one into
 * a graph.  Nothing attached: nothing to do, success.  No counterpart in the
 * reference, whose runner loads its device binary per run
 * (lib/Runtime/Execution/NativeExecutionRunner.cpp:372-528). */
uint32_t afir_hip_region_load(uint64_t handle);
/* Emit, compile and attach in one call, inside the process: the source of
 * afir_hip_region_emit_source is compiled for gfx950 by the runtime-compilation
 * library of the HIP runtime (libhiprtc, opened on first use), with the options
 * hipcc is given for the same source, so a host that has the runtime but no
 * hipcc still gets the program's own kernels instead of the interpreter.  Host
 * only (no device is touched; the code object is loaded at the first launch).
 * The code object is also copied to image_out when it fits `capacity` (a caller
 * that keeps artifacts), and its size stored in *image_len; both may be null.
 * The reference compiles its generated sources with an external compiler
 * (lib/Runtime/Compilation/KernelCompiler.cpp); this is that step without one. */
uint32_t afir_hip_region_compile(uint64_t handle, void *image_out, size_t capacity, size_t *image_len);
/* prefer != 0: the attached code object runs even when the program is one of
 * the hand-tuned families (which otherwise keep their kernel).  Used for
 * artifacts compiled with explicit emit options and by tile searches, where
 * the emitted kernel is the thing under test.  No counterpart in the
 * reference, whose kernels are all generated. */
uint32_t afir_hip_region_prefer_code_object(uint64_t handle, int prefer);
/* Name of tiling field `index` ("" if out of range); valid until unregister. */
const char *afir_hip_region_tiling_field(uint64_t handle, int index);
uint32_t afir_hip_region_argument_bytes(uint64_t handle, const void *tiling, size_t tiling_len,
                                        size_t *bytes, int max_args);
uint32_t afir_hip_launch_region(uint64_t handle, uint32_t block_dim, void *stream, int num_args,
                                void *const *args, void *workspace, const void *tiling,
                                size_t tiling_len);

#ifdef __cplusplus
}
#endif
#endif /* AFIR_HIP_KERNELS_H */
