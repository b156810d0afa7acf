"""Python caller of the afirt_* C API (libAFIRRuntimeCAPI.so, HIP backend).

Same entry points as the reference's python/runtime package
(executor.py:128-300, compiler.py:68-175, tiling_schema.py:17-128), so scripts
written against it read the same here:

    from ascend_mlir_amd.runtime import compile_kernel, execute_kernel, TilingSchema

The library is found through $AFIRT_CAPI_LIB (as in python/runtime/utils.py:60-91)
or next to this package.  Nothing here computes: arrays go to the GPU through
the C API and come back.
"""
from .capi import (CompilerError, ExecutorError, MAGIC_ELF_AICUBE, MAGIC_ELF_AIVEC,
                   capi_library_path, load_capi)
from .compiler import KernelCompiler, BishengCompiler, compile_kernel, read_binary
from .executor import HipRuntime, AscendRuntime, KernelExecutor, execute_kernel
from .tiling_schema import TilingSchema

__all__ = ["CompilerError", "ExecutorError", "MAGIC_ELF_AICUBE", "MAGIC_ELF_AIVEC",
           "capi_library_path", "load_capi", "KernelCompiler", "BishengCompiler",
           "compile_kernel", "read_binary", "HipRuntime", "AscendRuntime", "KernelExecutor",
           "execute_kernel", "TilingSchema"]
