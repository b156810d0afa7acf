"""Matmul with transposed and batched operands (linalg.matmul_transpose_a / _b,
linalg.batch_matmul*: lib/Conversion/MarkStructuredOps/AnnotateMixMatmulSemanticsPass.cpp:244-256)
as region programs on the GPU, against the region oracle.  Operands are small integers, so every
product and partial sum is exact in float32 and any summation order must give the oracle's
bits (the reference's own trick, test/tools/runtime known-answer tests); one case per layout
also runs on random operands within the matmul tolerance.  Needs a GPU."""
import subprocess
import os

import numpy as np
import pytest

from oracle import afir_oracle as O
from oracle import region_oracle as RO
from tests import mlir_cases as MC
from tests import region_cases as RC

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TR = os.path.join(ROOT, "ascend-mlir_amd", "bin", "afir-translate")


@pytest.fixture(scope="module")
def H(pkg):
    from ascend_mlir_amd import hip_kernels as H
    H.load()
    return H


def _program(rank, ty, flags, epilogue):
    """ty 'bf16': everything bf16; 'f16': f16 operands, float32 bias and output."""
    out_ty = "bf16" if ty == "bf16" else "f32"
    args = f"arg in {ty} {rank}\narg in {ty} {rank}\n"
    nin = 2
    if epilogue:
        args += f"arg in {out_ty} 1\n"
        nin = 3
    args += f"arg out {out_ty} {rank}\n"
    size = " ".join(f"arg{nin}.{d}" for d in range(rank))
    body = f" matmul arg0 arg1{flags}\n"
    if epilogue:
        body += f" push arg2 d{rank - 1}\n add\n leaky 0.25\n"
    return RC.HEADER + args + f"segment {rank}\n size {size}\n outoff 0\n" + body + " store\nend\n"


def _operands(rng, ty, batch, m, k, n, ta, tb, integers):
    def draw(shape):
        x = rng.integers(-4, 5, shape).astype(np.float32) if integers else \
            (rng.standard_normal(shape) / np.sqrt(k)).astype(np.float32)
        return O.f32_to_bf16_bits(x) if ty == "bf16" else x.astype(np.float16)
    lead = (batch,) if batch else ()
    a = draw(lead + ((k, m) if ta else (m, k)))
    b = draw(lead + ((n, k) if tb else (k, n)))
    bias = rng.integers(-3, 4, (n,)).astype(np.float32)
    bias = O.f32_to_bf16_bits(bias) if ty == "bf16" else bias
    return a, b, bias


def _run(H, text, inputs, ty, out_shape):
    """Launches through the raw entry point into an output that sits between two guard bands:
    nothing outside the output may be written."""
    import torch
    def dev(x):
        t = torch.from_numpy(x.view(np.int16) if x.dtype == np.uint16 else x).cuda()
        return t.view(torch.bfloat16) if x.dtype == np.uint16 else t
    r = H.Region(text)
    assert r.kernel.startswith("matmul_add_leakyrelu")
    devs = [dev(x) for x in inputs]
    odt = torch.int16 if ty == "bf16" else torch.float32
    count = int(np.prod(out_shape))
    guard = 4096   # elements on either side; keeps the output 16-byte aligned
    buf = torch.full((count + 2 * guard,), 0x5a5a if ty == "bf16" else 12345.0, dtype=odt, device="cuda")
    out = buf[guard:guard + count]
    dims = [d for t in devs for d in t.shape] + list(out_shape)
    H._check(r.launch_raw([t.data_ptr() for t in devs] + [out.data_ptr()], H.pack_tiling(*dims), 0, 0, None))
    torch.cuda.synchronize()
    r.close()
    host = buf.cpu().numpy()
    sentinel = host[0]
    assert (host[:guard] == sentinel).all() and (host[guard + count:] == sentinel).all(), "write outside the output"
    got = host[guard:guard + count].reshape(out_shape)
    return got.view(np.uint16) if ty == "bf16" else got


SHAPES = [(128, 64, 128), (256, 192, 384), (136, 72, 264), (1000, 200, 40), (64, 8, 64),
          (77, 33, 19), (8, 1, 8), (130, 520, 130)]


@pytest.mark.parametrize("ty", ["bf16", "f16"])
@pytest.mark.parametrize("flags", ["", " ta", " tb", " ta tb"])
@pytest.mark.parametrize("m,k,n", SHAPES)
def test_transposed_operands_integer_known_answer_exact(H, ty, flags, m, k, n):
    rng = np.random.default_rng(m * 31 + k * 7 + n)
    ta, tb = "ta" in flags, "tb" in flags
    for epilogue in (False, True):
        a, b, bias = _operands(rng, ty, 0, m, k, n, ta, tb, True)
        inputs = [a, b] + ([bias] if epilogue else [])
        text = _program(2, ty, flags, epilogue)
        want = RO.evaluate(text, inputs, out_shape=(m, n))
        got = _run(H, text, inputs, ty, (m, n))
        assert got.tobytes() == want.tobytes(), (flags, epilogue)


@pytest.mark.parametrize("ty", ["bf16", "f16"])
@pytest.mark.parametrize("flags", [" ta", " tb", " ta tb"])
def test_large_transposed_products_take_the_direct_to_lds_kernel(H, ty, flags):
    """Whole 256 x 256 tiles, at least half as many as the chip has compute units: the transposed
    operand is transposed into scratch memory of the stream and the product runs on the kernel of
    the plain layout.  Small integers: exact, whatever the order of summation."""
    m, k, n = 3072, 512, 3072
    rng = np.random.default_rng(5)
    a, b, bias = _operands(rng, ty, 0, m, k, n, "ta" in flags, "tb" in flags, True)
    text = _program(2, ty, flags, True)
    want = RO.evaluate(text, [a, b, bias], out_shape=(m, n))
    got = _run(H, text, [a, b, bias], ty, (m, n))
    assert H.last_launch()["kernel"].startswith("matmul_bias_leakyrelu_dma"), H.last_launch()
    assert got.tobytes() == want.tobytes()
    # twice in a row on the same stream: the scratch memory of the first call is free again
    got = _run(H, text, [a, b, bias], ty, (m, n))
    assert got.tobytes() == want.tobytes()


@pytest.mark.parametrize("ty", ["bf16", "f16"])
@pytest.mark.parametrize("flags,batch,m,k,n", [(f, b, m, k, n) for f in ("", " ta", " tb")
                                               for (b, m, k, n) in ((16, 256, 512, 2048), (6, 512, 256, 3072))] +
                         [(" ta tb", 16, 512, 4096, 1024)])
def test_large_batched_products_take_the_direct_to_lds_kernel(H, ty, flags, batch, m, k, n):
    """A batch of products of whole 256 x 256 tiles, at least half as many tiles in all as the chip
    has compute units, is one stack of tiles to the direct-to-LDS kernel: one tile row per product
    (16 x 256 rows), and two per product with the kernel's groups of four tile rows straddling
    products (6 x 512 rows).  Transposed operands are transposed per product first (both of them
    only where that pays: long K or large outputs).  Small integers: exact."""
    rng = np.random.default_rng(batch * 100 + m)
    a, b, bias = _operands(rng, ty, batch, m, k, n, "ta" in flags, "tb" in flags, True)
    text = _program(3, ty, flags, True)
    want = RO.evaluate(text, [a, b, bias], out_shape=(batch, m, n))
    got = _run(H, text, [a, b, bias], ty, (batch, m, n))
    assert H.last_launch()["kernel"].startswith("matmul_bias_leakyrelu_dma"), H.last_launch()
    assert "batched" in H.last_launch()["kernel"]
    assert got.tobytes() == want.tobytes()
    if not flags:                               # the same batch without bias and activation
        text = _program(3, ty, flags, False)
        want = RO.evaluate(text, [a, b], out_shape=(batch, m, n))
        got = _run(H, text, [a, b], ty, (batch, m, n))
        assert "batched" in H.last_launch()["kernel"] and got.tobytes() == want.tobytes()


@pytest.mark.parametrize("ty", ["bf16", "f16"])
@pytest.mark.parametrize("flags", ["", " ta", " tb"])
@pytest.mark.parametrize("batch,m,k,n", [(3, 128, 64, 128), (5, 136, 72, 40), (2, 77, 33, 19), (1, 64, 64, 64),
                                         (16, 256, 128, 256)])
def test_batched_products_integer_known_answer_exact(H, ty, flags, batch, m, k, n):
    rng = np.random.default_rng(batch * 1000 + m + k + n)
    ta, tb = "ta" in flags, "tb" in flags
    for epilogue in (False, True):
        a, b, bias = _operands(rng, ty, batch, m, k, n, ta, tb, True)
        inputs = [a, b] + ([bias] if epilogue else [])
        text = _program(3, ty, flags, epilogue)
        want = RO.evaluate(text, inputs, out_shape=(batch, m, n))
        got = _run(H, text, inputs, ty, (batch, m, n))
        assert got.tobytes() == want.tobytes(), (flags, epilogue)


@pytest.mark.parametrize("ty", ["bf16", "f16"])
@pytest.mark.parametrize("flags,batch", [(" ta", 0), (" tb", 0), (" ta tb", 0), ("", 4), (" tb", 4)])
def test_random_operands_within_the_matmul_tolerance(H, ty, flags, batch):
    """N(0, 1/sqrt(K)) operands, <= 1e-2 relative (atol 1e-5) as for C5, no NaN / inf the oracle lacks."""
    m, k, n = 384, 1024, 264
    rng = np.random.default_rng(11)
    a, b, bias = _operands(rng, ty, batch, m, k, n, "ta" in flags, "tb" in flags, False)
    rank = 3 if batch else 2
    shape = ((batch,) if batch else ()) + (m, n)
    text = _program(rank, ty, flags, True)
    want = RO.evaluate(text, [a, b, bias], out_shape=shape)
    got = _run(H, text, [a, b, bias], ty, shape)
    dt = "bf16" if ty == "bf16" else "f32"
    r = O.compare_outputs([(got, dt)], [(want, dt)], 1e-5, 1e-2)
    assert r["passed"], r
    assert O.nonfinite_mismatches(got, want, dt) == 0


def test_translated_graphs_run(H):
    """MLIR -> program -> kernel for one transposed and one batched graph."""
    rng = np.random.default_rng(3)
    for mlir, ty, batch, ta, tb in ((MC.MATMUL_TRANSPOSE_A_F16, "f16", 0, True, False),
                                    (MC.BATCH_MATMUL_TRANSPOSE_B_F16, "f16", 3, False, True),
                                    (MC.BATCH_MATMUL_BF16, "bf16", 2, False, False)):
        p = subprocess.run([TR, "-mlir-to-hip", "-"], input=mlir, capture_output=True, text=True)
        assert p.returncode == 0, p.stderr
        m, k, n = 136, 72, 264
        a, b, _ = _operands(rng, ty, batch, m, k, n, ta, tb, True)
        shape = ((batch,) if batch else ()) + (m, n)
        init = np.zeros(shape, np.uint16 if ty == "bf16" else np.float32)
        want = RO.evaluate(p.stdout, [a, b, init], out_shape=shape)
        got = _run(H, p.stdout, [a, b, init], ty, shape)
        assert got.tobytes() == want.tobytes()
