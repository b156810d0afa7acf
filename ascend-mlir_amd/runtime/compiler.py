"""Kernel source -> artifact, through afirt_compiler_* (reference:
python/runtime/compiler.py:68-175)."""
from __future__ import annotations

import ctypes
from pathlib import Path

from .capi import CompilerError, load_capi


class KernelCompiler:
    """Maps a fused-region source (.mlir text or a `hip_kernel=` descriptor)
    to an artifact naming a precompiled gfx950 kernel."""

    ARCH_VEC = "gfx950-vec"
    ARCH_CUBE = "gfx950-cube"

    def __init__(self, soc_version: str = "gfx950"):
        self.soc_version = soc_version

    def compile_and_link(self, src_file, output_dir, kernel_name: str, arch: str = ARCH_VEC,
                         opt_level: int = 3, verbose: bool = False) -> Path:
        src_file, output_dir = Path(src_file), Path(output_dir)
        output_dir.mkdir(parents=True, exist_ok=True)
        lib = load_capi()
        handle = lib.afirt_compiler_create(self.soc_version.encode(), arch.encode(), opt_level)
        if not handle:
            raise CompilerError("Failed to create compiler instance")
        try:
            buf = ctypes.create_string_buffer(4096)
            rc = lib.afirt_compiler_compile(handle, str(src_file.resolve()).encode(),
                                            str(output_dir.resolve()).encode(),
                                            kernel_name.encode(), buf, len(buf))
            if rc != 0:
                raise CompilerError(buf.value.decode(errors="replace"))
            path = Path(buf.value.decode())
        finally:
            lib.afirt_compiler_destroy(handle)
        if not path.exists():
            raise CompilerError(f"Binary file not generated: {path}")
        return path


BishengCompiler = KernelCompiler   # the reference's name for this role


def compile_kernel(src_file, output_dir, kernel_name: str, soc_version: str = "gfx950",
                   arch: str = KernelCompiler.ARCH_VEC, opt_level: int = 3,
                   verbose: bool = False) -> Path:
    return KernelCompiler(soc_version).compile_and_link(src_file, output_dir, kernel_name, arch,
                                                        opt_level, verbose)


def read_binary(path) -> bytes:
    return Path(path).read_bytes()
