"""Builds the gfx950 libraries in-tree with hipcc (cross-compiles without a GPU).

    python ascend-mlir_amd/build.py [--force]

Outputs (under ascend-mlir_amd/lib/):
    libafir_hip_kernels.so   fused kernels + launcher C ABI
"""
from __future__ import annotations

import concurrent.futures as cf
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "lib")
OBJ = os.path.join(HERE, "build")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
ARCH = "gfx950"

# -packed-fp32-ops off: the compiler must not form packed f32 instructions.
COMMON = ["-std=c++17", "-O3", "-fPIC", f"--offload-arch={ARCH}",
          "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
          "-Wall", "-Wno-unused-value", "-Wno-unknown-warning-option",
          "-I", os.path.join(ROOT, "include")]
# every f32 add/mul of the elementwise kernels stays a separate IEEE operation
STRICT = ["-ffp-contract=off"]

KERNEL_SOURCES = [
    ("kernels/eltwise.hip", STRICT),
    ("kernels/rowsum.hip", STRICT),
    ("kernels/transpose.hip", STRICT),
    ("kernels/gather.hip", STRICT),
    ("kernels/matmul.hip", []),
    ("kernels/matmul_dma.hip", []),
    ("capi/afir_hip_kernels.cpp", []),
]


def _run(cmd):
    p = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in p.stderr.splitlines()
                    if "packed-fp32-ops" not in l)
    if p.returncode != 0:
        raise RuntimeError("command failed: " + " ".join(cmd) + "\n" + err)
    if err.strip():
        sys.stderr.write(err + "\n")


def _compile(src, extra):
    obj = os.path.join(OBJ, src.replace("/", "_") + ".o")
    cmd = [HIPCC, *COMMON, *extra, "-x", "hip", "-c", os.path.join(CSRC, src), "-o", obj]
    _run(cmd)
    return obj


def build_kernels():
    os.makedirs(LIB, exist_ok=True)
    os.makedirs(OBJ, exist_ok=True)
    with cf.ThreadPoolExecutor(max_workers=min(8, len(KERNEL_SOURCES))) as ex:
        objs = list(ex.map(lambda a: _compile(*a), KERNEL_SOURCES))
    out = os.path.join(LIB, "libafir_hip_kernels.so")
    _run([HIPCC, "-shared", "-fPIC", f"--offload-arch={ARCH}", "-o", out, *objs])
    return out


def build_all():
    return [build_kernels()]


if __name__ == "__main__":
    for path in build_all():
        print("built", os.path.relpath(path, ROOT))
