/*
 * afirt_runtime.h — C API of libAFIRRuntimeCAPI.so for the HIP backend.
 *
 * Same symbols, argument meaning and error behaviour as the reference's
 * include/CAPI/Runtime.h:17-101 (implementation lib/CAPI/Runtime/Runtime.cpp:
 * 288-481), so that its ctypes caller (python/runtime/executor.py:128-241,
 * python/runtime/compiler.py:38-61) and its C++ caller
 * (test/tools/runtime/test_capi_runtime.cpp:111-191) bind this library
 * unchanged: point AFIRT_CAPI_LIB at it (python/runtime/utils.py:60-91).
 *
 * What differs behind the symbols, by necessity of the target:
 *   - "compile" maps a kernel source (MLIR text of a fused region, or a
 *     descriptor naming a kernel family) to an artifact that names one of the
 *     precompiled gfx950 kernels; out_bin_path is <output_dir>/<name>.hipk and
 *     <output_dir>/out/manifest.txt is written beside it;
 *   - "binary" passed to afirt_executor_run is the content of that .hipk file;
 *   - the executor runs on the GPU (hipSetDevice(device_id) at initialize),
 *     not on a simulator;
 *   - the API still carries no shapes: the executor takes them from the tiling
 *     bytes (fields dim_arg<A>_<D>, include/afir_hip_kernels.h) and rejects
 *     buffers whose byte counts do not match, instead of guessing a dtype.
 *
 * Return 0 on success, non-zero on error; messages are NUL-terminated and
 * truncated into the caller's buffer.  All data pointers are caller-owned host
 * memory, copied in and out.  The API takes no locks.
 */
#ifndef AFIRT_RUNTIME_H
#define AFIRT_RUNTIME_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct AfirtCompiler_s *AfirtCompiler;
typedef struct AfirtExecutor_s *AfirtExecutor;

/* include/CAPI/Runtime.h:24-29.  soc_version defaults to "gfx950"; arch and
 * opt_level are accepted and recorded (arch containing "cube" marks the
 * artifact kind as cube, as the reference derives it). */
AfirtCompiler afirt_compiler_create(const char *soc_version, const char *arch, int opt_level);
void afirt_compiler_destroy(AfirtCompiler compiler);

/* include/CAPI/Runtime.h:31-40.  On error the message is written into
 * out_bin_path. */
int afirt_compiler_compile(AfirtCompiler compiler, const char *src_file, const char *output_dir,
                           const char *kernel_name, char *out_bin_path, size_t buf_len);

/* include/CAPI/Runtime.h:46-54. */
AfirtExecutor afirt_executor_create(void);
void afirt_executor_destroy(AfirtExecutor executor);
int afirt_executor_initialize(AfirtExecutor executor, int device_id, char *err_buf, size_t err_len);

/* include/CAPI/Runtime.h:56-84.  magic: 0x41415246 or 0x41494343, anything
 * else is an error, as in the reference. */
int afirt_executor_run(AfirtExecutor executor, const uint8_t *binary_data, size_t binary_len,
                       const char *function_name, int num_inputs, const void **input_ptrs,
                       const size_t *input_bytes, int num_outputs, void **output_ptrs,
                       const size_t *output_bytes, const uint8_t *tiling_data, size_t tiling_len,
                       int block_dim, uint32_t magic, char *err_buf, size_t err_len);

/* include/CAPI/Runtime.h:86-97. */
int afirt_executor_run_file(AfirtExecutor executor, const char *binary_path,
                            const char *function_name, int num_inputs, const void **input_ptrs,
                            const size_t *input_bytes, int num_outputs, void **output_ptrs,
                            const size_t *output_bytes, const uint8_t *tiling_data,
                            size_t tiling_len, int block_dim, uint32_t magic, char *err_buf,
                            size_t err_len);

/* No counterpart in the reference.  What the executor's last successful run
 * launched: the kernel's device time in ns (HIP events around the launch; the
 * reference reports its simulator's cycle count through trace.json only), the
 * number of workgroups and lanes per workgroup of the last kernel, and its name
 * (truncated into kernel_name).  Any out pointer may be NULL.  Returns non-zero
 * when there has been no such run.
 *
 * block_dim of the two run calls above is the reference's unit, a number of
 * Ascend AI cores (its callers pass 1, 8 and 40).  It does not size the HIP
 * grid: the launcher does, for the device's compute units.  A process that
 * really means workgroups sets AFIR_HIP_HONOUR_BLOCK_DIM=1. */
int afirt_executor_last_launch(AfirtExecutor executor, int64_t *kernel_ns, uint32_t *workgroups,
                               uint32_t *threads, char *kernel_name, size_t name_len);

#ifdef __cplusplus
}
#endif
#endif /* AFIRT_RUNTIME_H */
