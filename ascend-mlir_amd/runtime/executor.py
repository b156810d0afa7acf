"""Kernel execution through afirt_executor_* (reference:
python/runtime/executor.py:128-300)."""
from __future__ import annotations

import ctypes
from typing import List, Optional, Sequence, Tuple

import numpy as np

from .capi import ExecutorError, MAGIC_ELF_AICUBE, MAGIC_ELF_AIVEC, load_capi


class HipRuntime:
    MAGIC_ELF_AIVEC = MAGIC_ELF_AIVEC
    MAGIC_ELF_AICUBE = MAGIC_ELF_AICUBE

    def __init__(self, soc_version: str = "gfx950"):
        self.soc_version = soc_version
        self._initialized = False
        self._handle = load_capi().afirt_executor_create()
        if not self._handle:
            raise ExecutorError("Failed to create executor instance")

    def __del__(self):
        if getattr(self, "_handle", None):
            try:
                load_capi().afirt_executor_destroy(self._handle)
            except Exception:
                pass
            self._handle = None

    def set_device(self, device_id: int = 0):
        err = ctypes.create_string_buffer(1024)
        rc = load_capi().afirt_executor_initialize(self._handle, device_id, err, len(err))
        if rc != 0:
            raise ExecutorError(err.value.decode(errors="replace"))
        self._initialized = True

    def run(self, binary_data: bytes, function_name: str, inputs: Sequence[np.ndarray],
            outputs: List[np.ndarray], tiling_data: Optional[bytes] = None, block_dim: int = 1,
            magic: int = MAGIC_ELF_AIVEC) -> List[np.ndarray]:
        """block_dim keeps the reference's meaning and default (a number of Ascend AI cores,
        python/runtime/executor.py:183): it is recorded, and the kernel's launcher sizes the HIP
        grid for the device.  AFIR_HIP_HONOUR_BLOCK_DIM=1 in the environment makes a positive
        block_dim the number of workgroups instead."""
        lib = load_capi()
        vp, sz = ctypes.c_void_p, ctypes.c_size_t
        bin_arr = (ctypes.c_uint8 * max(len(binary_data), 1)).from_buffer_copy(
            binary_data if binary_data else b"\0")
        in_bufs = [np.ascontiguousarray(x) for x in inputs]
        out_bufs = [np.ascontiguousarray(x) for x in outputs]
        in_ptrs = (vp * max(len(in_bufs), 1))(*[x.ctypes.data for x in in_bufs])
        in_bytes = (sz * max(len(in_bufs), 1))(*[x.nbytes for x in in_bufs])
        out_ptrs = (vp * max(len(out_bufs), 1))(*[x.ctypes.data for x in out_bufs])
        out_bytes = (sz * max(len(out_bufs), 1))(*[x.nbytes for x in out_bufs])
        if tiling_data:
            til = (ctypes.c_uint8 * len(tiling_data)).from_buffer_copy(tiling_data)
            til_ptr, til_len = ctypes.cast(til, ctypes.POINTER(ctypes.c_uint8)), len(tiling_data)
        else:
            til_ptr, til_len = ctypes.cast(None, ctypes.POINTER(ctypes.c_uint8)), 0
        err = ctypes.create_string_buffer(1024)
        rc = lib.afirt_executor_run(
            self._handle, ctypes.cast(bin_arr, ctypes.POINTER(ctypes.c_uint8)),
            len(binary_data), function_name.encode(), len(in_bufs), in_ptrs, in_bytes,
            len(out_bufs), out_ptrs, out_bytes, til_ptr, til_len, block_dim, magic, err, len(err))
        if rc != 0:
            raise ExecutorError(err.value.decode(errors="replace"))
        for dst, src in zip(outputs, out_bufs):
            if dst is not src:
                dst[...] = src
        return outputs


    def last_launch(self) -> dict:
        """Device time and grid of the last run's kernel (afirt_executor_last_launch)."""
        ns, wg, th = ctypes.c_int64(0), ctypes.c_uint32(0), ctypes.c_uint32(0)
        name = ctypes.create_string_buffer(128)
        if load_capi().afirt_executor_last_launch(self._handle, ctypes.byref(ns), ctypes.byref(wg),
                                                  ctypes.byref(th), name, len(name)) != 0:
            raise ExecutorError("no kernel has run on this executor")
        return {"kernel_ns": ns.value, "workgroups": wg.value, "threads": th.value,
                "kernel": name.value.decode(errors="replace")}


AscendRuntime = HipRuntime   # the reference's name for this role


class KernelExecutor:
    def __init__(self, soc_version: str = "gfx950", device_id: int = 0):
        self.runtime = HipRuntime(soc_version)
        self.device_id = device_id
        self._initialized = False

    def initialize(self):
        self.runtime.set_device(self.device_id)
        self._initialized = True

    def execute(self, binary_data, function_name, inputs, outputs, tiling_data=None,
                block_dim: int = 1, magic: int = MAGIC_ELF_AIVEC):
        if not self._initialized:
            self.initialize()
        return self.runtime.run(binary_data, function_name, inputs, outputs, tiling_data,
                                block_dim, magic)


def execute_kernel(binary_data: bytes, function_name: str, inputs: Sequence[np.ndarray],
                   output_shapes: Sequence[Tuple[int, ...]], tiling_data: Optional[bytes] = None,
                   soc_version: str = "gfx950", device_id: int = 0, dtype=np.float32):
    outputs = [np.zeros(shape, dtype=dtype) for shape in output_shapes]
    return KernelExecutor(soc_version, device_id).execute(binary_data, function_name, inputs,
                                                          outputs, tiling_data)
