"""ctypes binding of the fused-kernel C ABI (include/afir_hip_kernels.h).

Tensors are torch CUDA(ROCm) tensors used purely as device buffers; every
function launches on torch's current stream unless `stream` (a raw
hipStream_t value) is given, and returns the output tensor.  Nothing here
computes on the host.
"""
from __future__ import annotations

import ctypes
import os
import struct

from . import KERNELS_LIB

_HERE = os.path.dirname(os.path.abspath(__file__))


class AfirHipError(RuntimeError):
    pass


class _KernelInfo(ctypes.Structure):
    _fields_ = [("name", ctypes.c_char_p), ("symbol", ctypes.c_char_p),
                ("num_inputs", ctypes.c_int), ("num_outputs", ctypes.c_int),
                ("num_tiling_fields", ctypes.c_int),
                ("tiling_fields", ctypes.POINTER(ctypes.c_char_p)),
                ("signature", ctypes.c_char_p)]


EXPORTED_SYMBOLS = [
    "afir_hip_last_error",
    "afir_hip_launch_fused_add_mul",
    "afir_hip_launch_broadcast_add_reducesum",
    "afir_hip_launch_broadcast_add_reducesum_noalloc",
    "afir_hip_launch_relu_broadcast_add_transpose",
    "afir_hip_launch_gather_scale_shift",
    "afir_hip_launch_matmul_add_leakyrelu",
    "afir_hip_kernel_count",
    "afir_hip_kernel_info",
    "afir_hip_find_kernel",
    "afir_hip_launch",
    "afir_hip_argument_bytes",
    "afir_hip_region_register",
    "afir_hip_region_unregister",
    "afir_hip_region_info",
    "afir_hip_region_tiling_field",
    "afir_hip_region_kernel",
    "afir_hip_region_route",
    "afir_hip_region_emit_source",
    "afir_hip_region_attach_code_object",
    "afir_hip_region_compile",
    "afir_hip_region_load",
    "afir_hip_region_prefer_code_object",
    "afir_hip_region_argument_bytes",
    "afir_hip_launch_region",
    "afir_hip_last_launch",
]

_lib = None


def load():
    """dlopen the kernel library; raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(KERNELS_LIB):
        raise AfirHipError(
            f"{KERNELS_LIB} is missing: build it with "
            "`python ascend-mlir_amd/build.py` (there is no CPU fallback)")
    L = ctypes.CDLL(KERNELS_LIB)
    vp, u32 = ctypes.c_void_p, ctypes.c_uint32
    L.afir_hip_last_error.restype = ctypes.c_char_p
    L.afir_hip_last_launch.restype = ctypes.c_char_p
    L.afir_hip_last_launch.argtypes = [ctypes.POINTER(u32), ctypes.POINTER(u32)]
    for name, nptr in [("afir_hip_launch_fused_add_mul", 5),
                       ("afir_hip_launch_broadcast_add_reducesum", 5),
                       ("afir_hip_launch_broadcast_add_reducesum_noalloc", 5),
                       ("afir_hip_launch_relu_broadcast_add_transpose", 5),
                       ("afir_hip_launch_gather_scale_shift", 7),
                       ("afir_hip_launch_matmul_add_leakyrelu", 6)]:
        fn = getattr(L, name)
        fn.restype = u32
        fn.argtypes = [u32, vp] + [vp] * nptr
    L.afir_hip_kernel_count.restype = ctypes.c_int
    L.afir_hip_kernel_info.restype = ctypes.POINTER(_KernelInfo)
    L.afir_hip_kernel_info.argtypes = [ctypes.c_int]
    L.afir_hip_find_kernel.restype = ctypes.POINTER(_KernelInfo)
    L.afir_hip_find_kernel.argtypes = [ctypes.c_char_p]
    L.afir_hip_launch.restype = u32
    L.afir_hip_launch.argtypes = [ctypes.c_char_p, u32, vp, ctypes.c_int,
                                  ctypes.POINTER(vp), vp, vp, ctypes.c_size_t]
    _lib = L
    return L


def last_launch() -> dict:
    """The kernel this thread launched last through the library, and its grid."""
    wg, th = ctypes.c_uint32(0), ctypes.c_uint32(0)
    name = load().afir_hip_last_launch(ctypes.byref(wg), ctypes.byref(th))
    return {"kernel": (name or b"").decode(), "workgroups": wg.value, "threads": th.value}


def kernel_table():
    L = load()
    out = []
    for i in range(L.afir_hip_kernel_count()):
        k = L.afir_hip_kernel_info(i).contents
        out.append({
            "name": k.name.decode(), "symbol": k.symbol.decode(),
            "num_inputs": k.num_inputs, "num_outputs": k.num_outputs,
            "tiling_fields": [k.tiling_fields[j].decode()
                              for j in range(k.num_tiling_fields)],
            "signature": k.signature.decode()})
    return out


def pack_tiling(*fields) -> bytes:
    return struct.pack("<%dq" % len(fields), *[int(f) for f in fields])


def f32_bits(x: float) -> int:
    return struct.unpack("<I", struct.pack("<f", x))[0]


def _check(rc):
    if rc != 0:
        raise AfirHipError(f"rc={rc}: {load().afir_hip_last_error().decode()}")


def _stream(stream):
    if stream is not None:
        return ctypes.c_void_p(stream)
    import torch
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr())


def _dev(t, dtype, what):
    import torch
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise AfirHipError(f"{what}: expected a device tensor")
    if t.dtype != dtype:
        raise AfirHipError(f"{what}: expected {dtype}, got {t.dtype}")
    if not t.is_contiguous():
        raise AfirHipError(f"{what}: expected a contiguous tensor")
    return t


def launch_raw(symbol: str, block_dim: int, stream, ptrs, tiling: bytes):
    """Call a launcher symbol with raw device addresses (ints)."""
    L = load()
    fn = getattr(L, symbol)
    buf = ctypes.create_string_buffer(tiling, len(tiling))
    args = [ctypes.c_void_p(p) for p in ptrs]
    return fn(ctypes.c_uint32(block_dim), _stream(stream), *args,
              ctypes.cast(buf, ctypes.c_void_p))


def fused_add_mul(a, b, out=None, block_dim=0, stream=None):
    import torch
    _dev(a, torch.float32, "a"); _dev(b, torch.float32, "b")
    if a.shape != b.shape:
        raise AfirHipError("fused_add_mul: a and b must have the same shape")
    if out is None:
        out = torch.empty_like(a)
    _dev(out, torch.float32, "out")
    rows = a.shape[0] if a.dim() > 0 else 1
    cols = a.numel() // rows if rows else 0
    _check(launch_raw("afir_hip_launch_fused_add_mul", block_dim, stream,
                      [a.data_ptr(), b.data_ptr(), out.data_ptr(), 0],
                      pack_tiling(rows, cols)))
    return out


def broadcast_add_reducesum(x, bias, out=None, block_dim=0, stream=None):
    import torch
    _dev(x, torch.float32, "x"); _dev(bias, torch.float32, "bias")
    m, n = x.shape
    if bias.shape != (n,):
        raise AfirHipError("broadcast_add_reducesum: bias must have shape [N]")
    if out is None:
        out = torch.empty((m,), dtype=torch.float32, device=x.device)
    _dev(out, torch.float32, "out")
    _check(launch_raw("afir_hip_launch_broadcast_add_reducesum", block_dim, stream,
                      [x.data_ptr(), bias.data_ptr(), out.data_ptr(), 0],
                      pack_tiling(m, n)))
    return out


def relu_broadcast_add_transpose(x, c, out=None, block_dim=0, stream=None):
    import torch
    _dev(x, torch.float16, "x"); _dev(c, torch.float16, "c")
    b, m, n = x.shape
    if c.shape != (n,):
        raise AfirHipError("relu_broadcast_add_transpose: c must have shape [N]")
    if out is None:
        out = torch.empty((b, n, m), dtype=torch.float16, device=x.device)
    _dev(out, torch.float16, "out")
    _check(launch_raw("afir_hip_launch_relu_broadcast_add_transpose", block_dim, stream,
                      [x.data_ptr(), c.data_ptr(), out.data_ptr(), 0],
                      pack_tiling(b, m, n)))
    return out


def gather_scale_shift(table, indices, scale, shift, out=None, workspace=None,
                       block_dim=0, stream=None):
    import torch
    _dev(table, torch.float16, "table"); _dev(indices, torch.int32, "indices")
    _dev(scale, torch.float16, "scale"); _dev(shift, torch.float16, "shift")
    v, d = table.shape
    (r,) = indices.shape
    if scale.shape != (d,) or shift.shape != (d,):
        raise AfirHipError("gather_scale_shift: scale/shift must have shape [D]")
    if out is None:
        out = torch.empty((r, d), dtype=torch.float16, device=table.device)
    _dev(out, torch.float16, "out")
    ws = workspace.data_ptr() if workspace is not None else 0
    _check(launch_raw("afir_hip_launch_gather_scale_shift", block_dim, stream,
                      [table.data_ptr(), indices.data_ptr(), scale.data_ptr(),
                       shift.data_ptr(), out.data_ptr(), ws],
                      pack_tiling(v, d, r)))
    return out


def matmul_add_leakyrelu(a, b, bias, alpha=0.01, out=None, block_dim=0, stream=None):
    import torch
    _dev(a, torch.bfloat16, "a"); _dev(b, torch.bfloat16, "b")
    _dev(bias, torch.bfloat16, "bias")
    m, k = a.shape
    k2, n = b.shape
    if k != k2 or bias.shape != (n,):
        raise AfirHipError("matmul_add_leakyrelu: shape mismatch")
    if out is None:
        out = torch.empty((m, n), dtype=torch.bfloat16, device=a.device)
    _dev(out, torch.bfloat16, "out")
    _check(launch_raw("afir_hip_launch_matmul_add_leakyrelu", block_dim, stream,
                      [a.data_ptr(), b.data_ptr(), bias.data_ptr(), out.data_ptr(), 0],
                      pack_tiling(m, k, n, f32_bits(alpha))))
    return out


def prepare(symbol: str, ptrs, tiling: bytes, block_dim: int = 0, stream=None):
    """Pre-marshal one launch; returns a zero-argument callable that issues it
    (used by tight loops such as the benchmark to keep host overhead down).
    The stream is captured now."""
    L = load()
    fn = getattr(L, symbol)
    buf = ctypes.create_string_buffer(tiling, len(tiling))
    args = [ctypes.c_uint32(block_dim), _stream(stream)]
    args += [ctypes.c_void_p(p) for p in ptrs]
    args.append(ctypes.cast(buf, ctypes.c_void_p))

    def call(_fn=fn, _args=tuple(args), _keep=buf):
        rc = _fn(*_args)
        if rc:
            _check(rc)
    return call


# ---- fused-region programs ---------------------------------------------------

_TORCH_TYPES = None


def _torch_type(name):
    global _TORCH_TYPES
    import torch
    if _TORCH_TYPES is None:
        _TORCH_TYPES = {"f16": torch.float16, "bf16": torch.bfloat16, "f32": torch.float32,
                        "i32": torch.int32, "i64": torch.int64, "i16": torch.int16}
    return _TORCH_TYPES[name]


HIPCC_REGION_FLAGS = ["--genco", "--offload-arch=gfx950", "-O3", "-nogpuinc", "-ffp-contract=off",
                      "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def compile_region_source(source: str, cache_dir: str = None) -> bytes:
    """HIP source of a region (Region.emit_source, afir-translate
    --emit-hip-source) -> code object bytes.  Raises AfirHipError when hipcc is
    missing or rejects the source."""
    import hashlib
    import shutil
    import subprocess
    import tempfile
    cache_dir = cache_dir or os.path.join(_HERE, "lib", "region_cache")
    key = hashlib.sha256(("\n".join(HIPCC_REGION_FLAGS) + "\n" + source).encode()).hexdigest()[:24]
    path = os.path.join(cache_dir, key + ".hsaco")
    if os.path.exists(path):
        with open(path, "rb") as f:
            return f.read()
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        raise AfirHipError("hipcc not found: cannot compile a region kernel")
    os.makedirs(cache_dir, exist_ok=True)
    with tempfile.TemporaryDirectory() as tmp:
        src = os.path.join(tmp, "region.hip")
        obj = os.path.join(tmp, "region.hsaco")
        with open(src, "w") as f:
            f.write(source)
        p = subprocess.run([hipcc, *HIPCC_REGION_FLAGS, "-o", obj, src], capture_output=True, text=True)
        if p.returncode != 0:
            raise AfirHipError("hipcc rejected the region source:\n" + p.stderr[-2000:])
        with open(obj, "rb") as f:
            image = f.read()
    tmp_path = path + f".{os.getpid()}.tmp"
    with open(tmp_path, "wb") as f:
        f.write(image)
    os.replace(tmp_path, path)
    return image


class Region:
    """A registered fused-region program (afir_hip_region_register)."""

    def __init__(self, text: str):
        L = load()
        u64 = ctypes.c_uint64
        L.afir_hip_region_register.restype = ctypes.c_uint32
        L.afir_hip_region_register.argtypes = [ctypes.c_char_p, ctypes.c_size_t, ctypes.POINTER(u64)]
        L.afir_hip_region_unregister.argtypes = [u64]
        L.afir_hip_region_info.argtypes = [u64] + [ctypes.POINTER(ctypes.c_int)] * 3
        L.afir_hip_region_tiling_field.restype = ctypes.c_char_p
        L.afir_hip_region_tiling_field.argtypes = [u64, ctypes.c_int]
        L.afir_hip_region_argument_bytes.argtypes = [u64, ctypes.c_void_p, ctypes.c_size_t,
                                                    ctypes.POINTER(ctypes.c_size_t), ctypes.c_int]
        L.afir_hip_launch_region.restype = ctypes.c_uint32
        L.afir_hip_launch_region.argtypes = [u64, ctypes.c_uint32, ctypes.c_void_p, ctypes.c_int,
                                             ctypes.POINTER(ctypes.c_void_p), ctypes.c_void_p,
                                             ctypes.c_void_p, ctypes.c_size_t]
        data = text.encode()
        h = u64(0)
        _check(L.afir_hip_region_register(data, len(data), ctypes.byref(h)))
        self.handle = h.value
        ni, no, nf = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
        _check(L.afir_hip_region_info(u64(self.handle), ctypes.byref(ni), ctypes.byref(no), ctypes.byref(nf)))
        self.num_inputs, self.num_outputs = ni.value, no.value
        self.tiling_fields = [L.afir_hip_region_tiling_field(u64(self.handle), i).decode()
                              for i in range(nf.value)]
        L.afir_hip_region_kernel.restype = ctypes.c_char_p
        L.afir_hip_region_kernel.argtypes = [u64]
        self.kernel = L.afir_hip_region_kernel(u64(self.handle)).decode()
        self.arg_types = [l.split()[2] for l in text.splitlines() if l.split()[:1] == ["arg"]]

    # ---- kernels compiled for this program ----

    def emit_source(self) -> str:
        """HIP source of the kernels specialised for this program."""
        L = load()
        L.afir_hip_region_emit_source.argtypes = [ctypes.c_uint64, ctypes.c_char_p, ctypes.c_size_t,
                                                  ctypes.POINTER(ctypes.c_size_t)]
        n = ctypes.c_size_t(0)
        _check(L.afir_hip_region_emit_source(ctypes.c_uint64(self.handle), None, 0, ctypes.byref(n)))
        buf = ctypes.create_string_buffer(n.value + 1)
        _check(L.afir_hip_region_emit_source(ctypes.c_uint64(self.handle), buf, n.value + 1, ctypes.byref(n)))
        return buf.value.decode()

    def attach_code_object(self, image: bytes):
        L = load()
        L.afir_hip_region_attach_code_object.argtypes = [ctypes.c_uint64, ctypes.c_char_p, ctypes.c_size_t]
        _check(L.afir_hip_region_attach_code_object(ctypes.c_uint64(self.handle), image, len(image)))
        L.afir_hip_region_kernel.restype = ctypes.c_char_p
        self.kernel = L.afir_hip_region_kernel(ctypes.c_uint64(self.handle)).decode()

    def prefer_code_object(self, prefer: bool = True):
        """Run the attached code object even where a hand-tuned family matches."""
        L = load()
        L.afir_hip_region_prefer_code_object.argtypes = [ctypes.c_uint64, ctypes.c_int]
        _check(L.afir_hip_region_prefer_code_object(ctypes.c_uint64(self.handle), 1 if prefer else 0))
        L.afir_hip_region_kernel.restype = ctypes.c_char_p
        self.kernel = L.afir_hip_region_kernel(ctypes.c_uint64(self.handle)).decode()
        return self

    def compile(self, cache_dir: str = None, in_process: bool = None):
        """Emit, compile and attach.  With hipcc (the default where it exists) the code
        object is kept in `cache_dir` (default: lib/region_cache beside the libraries)
        under the hash of its source, so a program is compiled once.  in_process=True, or
        no hipcc on this host: compiled inside the process by the HIP runtime's own
        compiler library (afir_hip_region_compile), nothing cached."""
        import shutil
        if in_process is None:
            in_process = not (shutil.which("hipcc") or os.path.exists("/opt/rocm/bin/hipcc"))
        if in_process:
            L = load()
            L.afir_hip_region_compile.restype = ctypes.c_uint32
            L.afir_hip_region_compile.argtypes = [ctypes.c_uint64, ctypes.c_void_p, ctypes.c_size_t,
                                                  ctypes.POINTER(ctypes.c_size_t)]
            n = ctypes.c_size_t(0)
            _check(L.afir_hip_region_compile(ctypes.c_uint64(self.handle), None, 0, ctypes.byref(n)))
            self.kernel = L.afir_hip_region_kernel(ctypes.c_uint64(self.handle)).decode()
            return self
        source = self.emit_source()
        self.attach_code_object(compile_region_source(source, cache_dir))
        return self

    def close(self):
        if self.handle:
            load().afir_hip_region_unregister(ctypes.c_uint64(self.handle))
            self.handle = 0

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def route(self, tiling: bytes) -> str:
        """"family", "compiled" or "interpreter": the kernels a launch with these
        shapes runs on (host only)."""
        L = load()
        L.afir_hip_region_route.restype = ctypes.c_char_p
        L.afir_hip_region_route.argtypes = [ctypes.c_uint64, ctypes.c_void_p, ctypes.c_size_t]
        buf = ctypes.create_string_buffer(tiling, len(tiling))
        got = L.afir_hip_region_route(ctypes.c_uint64(self.handle), buf, len(tiling)).decode()
        if not got:
            raise AfirHipError(L.afir_hip_last_error().decode())
        return got

    def argument_bytes(self, tiling: bytes):
        n = self.num_inputs + self.num_outputs
        out = (ctypes.c_size_t * n)()
        buf = ctypes.create_string_buffer(tiling, len(tiling))
        _check(load().afir_hip_region_argument_bytes(ctypes.c_uint64(self.handle), buf, len(tiling), out, n))
        return list(out)

    def launch_raw(self, ptrs, tiling: bytes, workspace=0, block_dim=0, stream=None):
        arr = (ctypes.c_void_p * len(ptrs))(*[ctypes.c_void_p(p) for p in ptrs])
        buf = ctypes.create_string_buffer(tiling, len(tiling))
        return load().afir_hip_launch_region(ctypes.c_uint64(self.handle), block_dim, _stream(stream),
                                             len(ptrs), arr, ctypes.c_void_p(workspace), buf, len(tiling))

    def prepare(self, ptrs, tiling: bytes, workspace=0, block_dim=0, stream=None):
        """Pre-marshal one launch; returns a zero-argument callable."""
        L = load()
        arr = (ctypes.c_void_p * len(ptrs))(*[ctypes.c_void_p(p) for p in ptrs])
        buf = ctypes.create_string_buffer(tiling, len(tiling))
        args = (ctypes.c_uint64(self.handle), ctypes.c_uint32(block_dim), _stream(stream), len(ptrs),
                arr, ctypes.c_void_p(workspace), ctypes.cast(buf, ctypes.c_void_p), len(tiling))

        def call(_fn=L.afir_hip_launch_region, _args=args, _keep=(arr, buf)):
            rc = _fn(*_args)
            if rc:
                _check(rc)
        return call

    def __call__(self, *inputs, out_shape, workspace=None, block_dim=0, stream=None):
        """inputs: device tensors in argument order; returns the output tensor."""
        import torch
        if len(inputs) != self.num_inputs:
            raise AfirHipError(f"region expects {self.num_inputs} inputs, got {len(inputs)}")
        for i, t in enumerate(inputs):
            _dev(t, _torch_type(self.arg_types[i]), f"region input {i}")
        out = torch.empty(tuple(out_shape), dtype=_torch_type(self.arg_types[-1]), device=inputs[0].device)
        dims = [d for t in inputs for d in t.shape] + list(out.shape)
        tiling = pack_tiling(*dims)
        ws = workspace.data_ptr() if workspace is not None else 0
        _check(self.launch_raw([t.data_ptr() for t in inputs] + [out.data_ptr()], tiling, ws,
                               block_dim, stream))
        return out
