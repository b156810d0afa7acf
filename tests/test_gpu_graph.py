"""The launch entry points recorded into a HIP graph and replayed: launch-bound
chains of small kernels are meant to be captured once and replayed.  Every replay,
with the program's own eager work and synchronisations between replays, must give
what the same launches give eagerly.  Needs a GPU."""
import numpy as np
import pytest

from tests import region_cases as RC

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


@pytest.fixture(scope="module")
def H(pkg):
    from ascend_mlir_amd import hip_kernels
    hip_kernels.load()
    assert torch.cuda.is_available(), "no GPU visible"
    return hip_kernels


def test_kernels_replay_from_a_captured_graph(H, tmp_path, monkeypatch):
    """(a + b) * b on the hand-tuned kernel, then relu(col) + x on a compiled region, then
    the row sums of a handful of long rows (the split / join pair) -- captured together."""
    monkeypatch.setenv("AFIR_HIP_REGION_GENERIC", "1")
    m, n = 96, 256
    gen = torch.Generator(device="cuda").manual_seed(3)

    def ints(shape, dtype):
        return torch.randint(-3, 4, shape, generator=gen, device="cuda", dtype=torch.int32).to(dtype)

    a, b = ints((m, n), torch.float32), ints((m, n), torch.float32)
    ab = torch.empty_like(a)
    col, x = ints((n, 1), torch.float16), ints((m, n), torch.float16)
    y = torch.empty_like(x)
    long_rows = ints((2, 16 * 8192), torch.float16)
    row_term = ints((2,), torch.float16) * 2.0 ** -8        # 131072 of them stay inside the f16 range
    sums = torch.empty((2,), dtype=torch.float16, device="cuda")
    elementwise = H.Region(RC.RELU_COL_ADD).compile(str(tmp_path))
    row_sum = H.Region(RC.REDUCE_ROWBIAS).compile(str(tmp_path))

    def launches():
        return [
            H.prepare("afir_hip_launch_fused_add_mul", [a.data_ptr(), b.data_ptr(), ab.data_ptr(), 0], H.pack_tiling(m, n)),
            elementwise.prepare([col.data_ptr(), x.data_ptr(), y.data_ptr()], H.pack_tiling(n, 1, m, n, m, n)),
            row_sum.prepare([row_term.data_ptr(), long_rows.data_ptr(), sums.data_ptr()],
                            H.pack_tiling(2, 2, 16 * 8192, 2)),
        ]

    def eager():
        for call in launches():
            call()
        torch.cuda.synchronize()
        return ab.clone(), y.clone(), sums.clone()

    eager()                                   # modules loaded, kernels resolved
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for call in launches():               # prepared inside: the stream is the capturing one
            call()
    for replay in range(4):
        for t in (a, b, x, long_rows):        # eager work between replays: new inputs in the same buffers
            t.copy_(ints(tuple(t.shape), t.dtype))
        want = eager()
        for t in (ab, y, sums):
            t.fill_(7)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for got, expected, what in zip((ab, y, sums), want, ("add-mul", "region", "row sums")):
            assert torch.equal(got, expected), (replay, what)
    assert torch.equal(ab, (a + b) * b) and torch.equal(y, torch.relu(col.t()) + x)
    total = long_rows.float().sum(dim=1) + 16 * 8192 * row_term.float()
    assert bool(torch.isfinite(total.half()).all()) and torch.equal(sums, total.half())
    elementwise.close()
    row_sum.close()


def test_phased_kernels_replay_from_a_captured_graph(H):
    """The gather and the transpose on the kernels that hold their stores back by the device's
    real-time counter (the gather with rows left over: a second launch of the other kernel),
    captured together: the hold lives inside the kernels, so replays behave like eager launches."""
    gen = torch.Generator(device="cuda").manual_seed(5)
    rows, dim, nidx = 5000, 1024, 4099
    table = torch.randn((rows, dim), generator=gen, device="cuda").half()
    scale = torch.randn((dim,), generator=gen, device="cuda").half()
    shift = torch.randn((dim,), generator=gen, device="cuda").half()
    idx = torch.randint(0, rows, (nidx,), generator=gen, device="cuda", dtype=torch.int32)
    gathered = torch.empty((nidx, dim), dtype=torch.float16, device="cuda")
    b, m, n = 12, 1024, 1024
    x = torch.randn((b, m, n), generator=gen, device="cuda").half()
    c = torch.randn((n,), generator=gen, device="cuda").half()
    xt = torch.empty((b, n, m), dtype=torch.float16, device="cuda")

    def launches():
        return [
            H.prepare("afir_hip_launch_gather_scale_shift",
                      [table.data_ptr(), idx.data_ptr(), scale.data_ptr(), shift.data_ptr(), gathered.data_ptr(), 0],
                      H.pack_tiling(rows, dim, nidx)),
            H.prepare("afir_hip_launch_relu_broadcast_add_transpose", [x.data_ptr(), c.data_ptr(), xt.data_ptr(), 0],
                      H.pack_tiling(b, m, n)),
        ]

    def eager():
        for call in launches():
            call()
        torch.cuda.synchronize()
        return gathered.clone(), xt.clone()

    eager()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for call in launches():
            call()
    for replay in range(3):
        idx.copy_(torch.randint(0, rows, (nidx,), generator=gen, device="cuda", dtype=torch.int32))
        x.copy_(torch.randn((b, m, n), generator=gen, device="cuda").half())
        want = eager()
        gathered.fill_(7)
        xt.fill_(7)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for got, expected, what in zip((gathered, xt), want, ("gather", "transpose")):
            assert torch.equal(got, expected), (replay, what)
    # f32 multiply and add (the product of two halves is exact in f32), one rounding to f16
    assert torch.equal(gathered, (table[idx.long()].float() * scale.float() + shift.float()).half())
    assert torch.equal(xt, (torch.relu(x.float()) + c.float()).half().transpose(1, 2))


def test_phased_kernels_that_overlap_on_two_streams(H):
    """The gather, the transpose and the add-mul chain on the kernels that hold their stores back,
    launched on two streams at once, several times over: the kernels then share the chip, which
    the hold does not expect -- it may cost time, never results."""
    gen = torch.Generator(device="cuda").manual_seed(11)
    rows, dim, nidx = 4000, 1024, 16384
    table = torch.randn((rows, dim), generator=gen, device="cuda").half()
    scale = torch.randn((dim,), generator=gen, device="cuda").half()
    shift = torch.randn((dim,), generator=gen, device="cuda").half()
    idx = torch.randint(0, rows, (nidx,), generator=gen, device="cuda", dtype=torch.int32)
    b, m, n = 24, 1024, 512
    x = torch.randn((b, m, n), generator=gen, device="cuda").half()
    c = torch.randn((n,), generator=gen, device="cuda").half()
    p = torch.randn((2048, 4096), generator=gen, device="cuda")
    q = torch.randn((2048, 4096), generator=gen, device="cuda")
    want_g = (table[idx.long()].float() * scale.float() + shift.float()).half()
    want_t = (torch.relu(x.float()) + c.float()).half().transpose(1, 2).contiguous()
    want_e = (p + q) * q
    torch.cuda.synchronize()
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    for rep in range(5):
        got_g = torch.full((nidx, dim), 7, dtype=torch.float16, device="cuda")
        got_t = torch.full((b, n, m), 7, dtype=torch.float16, device="cuda")
        got_e = torch.full((2048, 4096), 7, dtype=torch.float32, device="cuda")
        torch.cuda.synchronize()
        H.gather_scale_shift(table, idx, scale, shift, out=got_g, stream=s1.cuda_stream)
        H.relu_broadcast_add_transpose(x, c, out=got_t, stream=s2.cuda_stream)
        H.fused_add_mul(p, q, out=got_e, stream=s1.cuda_stream)
        H.relu_broadcast_add_transpose(x, c, out=got_t, stream=s2.cuda_stream)
        H.gather_scale_shift(table, idx, scale, shift, out=got_g, stream=s2.cuda_stream)
        torch.cuda.synchronize()
        assert torch.equal(got_g, want_g), rep
        assert torch.equal(got_t, want_t), rep
        assert torch.equal(got_e, want_e), rep


def test_matmul_layouts_replay_from_a_captured_graph(H):
    """A large product with a transposed operand allocates scratch memory of its stream when it is
    launched eagerly; under a capture it may not, and keeps to the kernel that needs none.  A
    batch of products needs no scratch on either route.  Small integers: both routes give the
    same bits, and every replay must match the eager launches on the same inputs."""
    m, k, n, nb = 3072, 512, 3072, 8
    gen = torch.Generator(device="cuda").manual_seed(5)

    def ints(shape):
        return torch.randint(-3, 4, shape, generator=gen, device="cuda", dtype=torch.int32).to(torch.bfloat16)

    def program(rank, flags):
        size = " ".join(f"arg2.{d}" for d in range(rank))
        return (RC.HEADER + f"arg in bf16 {rank}\narg in bf16 {rank}\narg out bf16 {rank}\nsegment {rank}\n size {size}\n"
                f" outoff 0\n matmul arg0 arg1{flags}\n store\nend\n")
    at, b = ints((k, m)), ints((k, n))                      # A stored [K, M]
    ba, bb = ints((nb, 512, 256)), ints((nb, 256, 1024))    # 8 x 2 x 4 = 64 tiles: the register-staged kernel
    c, bc = torch.empty((m, n), dtype=torch.bfloat16, device="cuda"), torch.empty((nb, 512, 1024), dtype=torch.bfloat16, device="cuda")
    transposed, batched = H.Region(program(2, " ta")), H.Region(program(3, ""))

    def launches():
        return [transposed.prepare([at.data_ptr(), b.data_ptr(), c.data_ptr()], H.pack_tiling(k, m, k, n, m, n)),
                batched.prepare([ba.data_ptr(), bb.data_ptr(), bc.data_ptr()],
                                H.pack_tiling(nb, 512, 256, nb, 256, 1024, nb, 512, 1024))]

    def eager():
        names = []
        for call in launches():
            call()
            names.append(H.last_launch()["kernel"])
        torch.cuda.synchronize()
        return c.clone(), bc.clone(), names
    _, _, names = eager()
    assert names[0].startswith("matmul_bias_leakyrelu_dma"), names     # eagerly: transposed into scratch, then the direct kernel
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for call in launches():
            call()
        captured = H.last_launch()["kernel"]
    for replay in range(3):
        for t in (at, b, ba, bb):
            t.copy_(ints(tuple(t.shape)))
        want_c, want_bc, _ = eager()
        c.fill_(7)
        bc.fill_(7)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(c, want_c) and torch.equal(bc, want_bc), replay
    assert torch.equal(c, (at.float().t() @ b.float()).bfloat16())      # exact sums, one rounding to bf16
    assert captured  # (whichever kernel the batch took: it allocates nothing)
    transposed.close()
    batched.close()
