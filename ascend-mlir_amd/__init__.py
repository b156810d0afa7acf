"""afir-hip: gfx950 fused kernels behind Ascend-MLIR's runtime boundary.

The directory name carries a hyphen, so import it by path (tests/conftest.py,
bench.py and __graft_entry__.py register it as `ascend_mlir_amd`).

    hip_kernels   ctypes binding of libafir_hip_kernels.so (device pointers)

There is no CPU fallback: every entry point raises if the HIP library has not
been built (python ascend-mlir_amd/build.py).
"""
import os

PACKAGE_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_DIR = os.path.join(PACKAGE_DIR, "lib")
KERNELS_LIB = os.path.join(LIB_DIR, "libafir_hip_kernels.so")

__all__ = ["PACKAGE_DIR", "LIB_DIR", "KERNELS_LIB"]
