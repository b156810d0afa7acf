"""ctypes binding of libafir_bench_probes.so (csrc/bench/probes.h): measurement
aids of the benchmark.  Not part of the drop-in: nothing else loads it."""
from __future__ import annotations

import ctypes
import os

from . import LIB_DIR

PROBES_LIB = os.path.join(LIB_DIR, "libafir_bench_probes.so")
MFMA_OPERAND_BYTES = 65536
MFMA_SINK_BYTES = 1 << 20

_lib = None


def load():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(PROBES_LIB):
        raise RuntimeError(f"{PROBES_LIB} is missing: build it with `python ascend-mlir_amd/build.py`")
    L = ctypes.CDLL(PROBES_LIB)
    vp, u32 = ctypes.c_void_p, ctypes.c_uint32
    for name, args in [("afir_bench_mfma_rate", [vp, vp, vp, u32, ctypes.POINTER(ctypes.c_uint64)]),
                       ("afir_bench_matmul_ablated", [vp, vp, vp, vp, vp, ctypes.c_int, ctypes.c_int,
                                                      ctypes.c_int, ctypes.c_int]),
                       ("afir_bench_copy", [vp, vp, vp, ctypes.c_size_t]),
                       ("afir_bench_copy_phased", [vp, vp, vp, ctypes.c_size_t]),
                       ("afir_bench_fill", [vp, vp, ctypes.c_size_t, u32]),
                       ("afir_bench_read", [vp, vp, vp, ctypes.c_size_t]),
                       ("afir_bench_tilecopy64", [vp, vp, vp, ctypes.c_int, ctypes.c_int, ctypes.c_int])]:
        fn = getattr(L, name)
        fn.restype = u32
        fn.argtypes = args
    _lib = L
    return L


def _stream():
    import torch
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _check(rc, what):
    if rc:
        raise RuntimeError(f"{what}: rc={rc}")


def mfma_rate(operands, iters=20000, repeats=3):
    """TFLOP/s at which the matrix cores retire bf16 MFMAs fed from registers, for the
    given operand values (a device tensor of >= 65536 bytes); best of `repeats`."""
    import torch
    L = load()
    if not operands.is_cuda or operands.numel() * operands.element_size() < MFMA_OPERAND_BYTES:
        raise RuntimeError("mfma_rate: need a device tensor of at least 65536 bytes")
    sink = torch.empty(MFMA_SINK_BYTES // 4, dtype=torch.float32, device=operands.device)
    flops = ctypes.c_uint64(0)
    _check(L.afir_bench_mfma_rate(_stream(), operands.data_ptr(), sink.data_ptr(), 200, ctypes.byref(flops)),
           "mfma_rate")
    torch.cuda.synchronize()
    best = 0.0
    for _ in range(repeats):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        _check(L.afir_bench_mfma_rate(_stream(), operands.data_ptr(), sink.data_ptr(), iters,
                                      ctypes.byref(flops)), "mfma_rate")
        e1.record()
        torch.cuda.synchronize()
        best = max(best, flops.value / (e0.elapsed_time(e1) * 1e-3) / 1e12)
    return best


def prepare(name, *args):
    """A zero-argument callable that issues probe `name` on the current stream."""
    L = load()
    fn = getattr(L, name)
    full = (_stream(),) + tuple(args)

    def call(_fn=fn, _args=full, _what=name):
        rc = _fn(*_args)
        if rc:
            _check(rc, _what)
    return call
