"""ctypes prototypes of the afirt_* symbols (include/afirt_runtime.h)."""
from __future__ import annotations

import ctypes
import os

from .. import LIB_DIR

MAGIC_ELF_AIVEC = 0x41415246
MAGIC_ELF_AICUBE = 0x41494343

EXPORTED_SYMBOLS = [
    "afirt_compiler_create", "afirt_compiler_destroy", "afirt_compiler_compile",
    "afirt_executor_create", "afirt_executor_destroy", "afirt_executor_initialize",
    "afirt_executor_run", "afirt_executor_run_file", "afirt_executor_last_launch",
]


class ExecutorError(RuntimeError):
    pass


class CompilerError(RuntimeError):
    pass


_lib = None


def capi_library_path() -> str:
    env = os.environ.get("AFIRT_CAPI_LIB")
    if env:
        return env
    return os.path.join(LIB_DIR, "libAFIRRuntimeCAPI.so")


def load_capi() -> ctypes.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    path = capi_library_path()
    if not os.path.exists(path):
        raise ExecutorError(f"{path} is missing: build it with "
                            "`python ascend-mlir_amd/build.py` (there is no CPU fallback)")
    L = ctypes.CDLL(path)
    vp, sz, cp = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_char_p
    L.afirt_compiler_create.restype = vp
    L.afirt_compiler_create.argtypes = [cp, cp, ctypes.c_int]
    L.afirt_compiler_destroy.restype = None
    L.afirt_compiler_destroy.argtypes = [vp]
    L.afirt_compiler_compile.restype = ctypes.c_int
    L.afirt_compiler_compile.argtypes = [vp, cp, cp, cp, cp, sz]
    L.afirt_executor_create.restype = vp
    L.afirt_executor_create.argtypes = []
    L.afirt_executor_destroy.restype = None
    L.afirt_executor_destroy.argtypes = [vp]
    L.afirt_executor_initialize.restype = ctypes.c_int
    L.afirt_executor_initialize.argtypes = [vp, ctypes.c_int, cp, sz]
    run_tail = [cp, ctypes.c_int, ctypes.POINTER(vp), ctypes.POINTER(sz), ctypes.c_int,
                ctypes.POINTER(vp), ctypes.POINTER(sz), ctypes.POINTER(ctypes.c_uint8), sz,
                ctypes.c_int, ctypes.c_uint32, cp, sz]
    L.afirt_executor_run.restype = ctypes.c_int
    L.afirt_executor_run.argtypes = [vp, ctypes.POINTER(ctypes.c_uint8), sz] + run_tail
    L.afirt_executor_run_file.restype = ctypes.c_int
    L.afirt_executor_run_file.argtypes = [vp, cp] + run_tail
    L.afirt_executor_last_launch.restype = ctypes.c_int
    L.afirt_executor_last_launch.argtypes = [vp, ctypes.POINTER(ctypes.c_int64), ctypes.POINTER(ctypes.c_uint32),
                                             ctypes.POINTER(ctypes.c_uint32), cp, sz]
    _lib = L
    return L
