"""The C-ABI library loads without a GPU and exports every declared symbol."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(afir[a-z_]*_[a-z_0-9]+)\s*\(", text)))


def test_kernel_library_exports_every_declared_symbol(pkg):
    from ascend_mlir_amd import hip_kernels as H
    L = H.load()
    names = _declared("afir_hip_kernels.h")
    assert set(H.EXPORTED_SYMBOLS) <= set(names)
    for n in names:
        assert hasattr(L, n), n


def test_registry_is_consistent(pkg):
    from ascend_mlir_amd import hip_kernels as H
    L = H.load()
    table = H.kernel_table()
    assert [k["name"] for k in table] == [
        "fused_add_mul", "broadcast_add_reducesum", "relu_broadcast_add_transpose",
        "gather_scale_shift", "matmul_add_leakyrelu"]
    for k in table:
        assert hasattr(L, k["symbol"])
        assert k["num_outputs"] == 1
        assert all(f.startswith("dim_arg") or f == "alpha_f32_bits" for f in k["tiling_fields"])
        info = L.afir_hip_find_kernel(k["name"].encode())
        assert info and info.contents.symbol.decode() == k["symbol"]
    assert not L.afir_hip_find_kernel(b"nope")
    assert not L.afir_hip_kernel_info(99)


def test_argument_errors_need_no_gpu(pkg):
    # validation happens on the host before any launch
    from ascend_mlir_amd import hip_kernels as H
    L = H.load()
    til = H.pack_tiling(4, 4)
    args = (ctypes.c_void_p * 3)(0, 0, 0)
    assert L.afir_hip_launch(b"nope", 0, None, 3, args, None, til, len(til)) == 3
    assert L.afir_hip_launch(b"fused_add_mul", 0, None, 3, args, None, til, 4) == 1
    assert L.afir_hip_launch(b"fused_add_mul", 0, None, 1, args, None, til, len(til)) == 1
    # null tensors with a non-empty shape are rejected, not launched
    assert L.afir_hip_launch(b"fused_add_mul", 0, None, 3, args, None, til, len(til)) == 1
    assert b"null" in L.afir_hip_last_error()
    neg = H.pack_tiling(-4, 4)
    assert L.afir_hip_launch(b"fused_add_mul", 0, None, 3, args, None, neg, len(neg)) == 1


def test_missing_library_fails_loudly(pkg, monkeypatch):
    from ascend_mlir_amd import hip_kernels as H
    monkeypatch.setattr(H, "_lib", None)
    monkeypatch.setattr(H, "KERNELS_LIB", "/nonexistent/libafir_hip_kernels.so")
    with pytest.raises(H.AfirHipError, match="no CPU fallback"):
        H.load()
