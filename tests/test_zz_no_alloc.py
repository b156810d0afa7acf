"""The row-sum entry point that allocates nothing
(afir_hip_launch_broadcast_add_reducesum_noalloc: partial sums in a device array
of the library) against the ordinary entry point, through the C ABI: two calls
in a row, the second on a smaller input, so that what the first call left in the
scratch array must not leak into the second."""
import ctypes

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

NOALLOC = "afir_hip_launch_broadcast_add_reducesum_noalloc"
PLAIN = "afir_hip_launch_broadcast_add_reducesum"


@pytest.fixture(scope="module")
def H(pkg):
    import torch
    from ascend_mlir_amd import hip_kernels
    hip_kernels.load()
    assert torch.cuda.is_available()
    return hip_kernels


def run(H, symbol, x, bias):
    import torch
    m, n = x.shape
    y = torch.full((m,), float("nan"), dtype=torch.float32, device="cuda")
    rc = H.launch_raw(symbol, 0, None, [x.data_ptr(), bias.data_ptr(), y.data_ptr(), 0], H.pack_tiling(m, n))
    assert rc == 0, (symbol, rc)
    torch.cuda.synchronize()
    return y.cpu().numpy()


def check_pair(H, m, n, seed):
    import torch
    rng = np.random.default_rng(seed)
    # small integers: every partial sum is exact in float32, so any order of addition gives the same bits
    xi = torch.from_numpy(rng.integers(-4, 5, (m, n)).astype(np.float32)).cuda()
    bi = torch.from_numpy(rng.integers(-4, 5, (n,)).astype(np.float32)).cuda()
    got, want = run(H, NOALLOC, xi, bi), run(H, PLAIN, xi, bi)
    assert got.tobytes() == want.tobytes(), (m, n)
    assert np.array_equal(got, (xi.double().sum(1) + bi.double().sum()).cpu().numpy().astype(np.float32))
    # uniform values: a float32 sum in another order, held to 1e-5 relative (plus the floor
    # of 1e-7 times the sum of the terms' magnitudes, for rows that cancel)
    xu = torch.from_numpy(rng.uniform(-1, 1, (m, n)).astype(np.float32)).cuda()
    bu = torch.from_numpy(rng.uniform(-1, 1, (n,)).astype(np.float32)).cuda()
    got, want = run(H, NOALLOC, xu, bu).astype(np.float64), run(H, PLAIN, xu, bu).astype(np.float64)
    scale = (xu.double() + bu.double()).abs().sum(1).cpu().numpy()
    assert np.all(np.abs(got - want) <= 1e-5 * np.abs(want) + 1e-7 * scale), (m, n)


def test_noalloc_rowsum_matches_the_ordinary_entry_point_on_two_calls_in_a_row(H):
    check_pair(H, 16, 1 << 20, seed=1)      # 16 rows x 128 chunks: 2048 partial sums in the scratch array
    check_pair(H, 7, 40000, seed=2)         # smaller: 7 rows x 5 chunks, the last one short
    check_pair(H, 1023, 16384, seed=3)      # the most rows of the split form, two chunks each
    check_pair(H, 512, 4096, seed=4)        # a shape that needs no scratch: the ordinary kernels
    check_pair(H, 3, 16388, seed=5)         # a last chunk of one vector


def test_noalloc_rowsum_refuses_what_does_not_fit_the_scratch_array(H):
    import torch
    m, n = 1000, 1 << 20                    # 1000 rows x 128 chunks = 128000 partial sums > 65536
    x = torch.zeros((8,), dtype=torch.float32, device="cuda")     # never read: the call launches nothing
    y = torch.full((m,), 7.0, dtype=torch.float32, device="cuda")
    rc = H.launch_raw(NOALLOC, 0, None, [x.data_ptr(), x.data_ptr(), y.data_ptr(), 0], H.pack_tiling(m, n))
    assert rc == 4                          # AFIR_HIP_E_NOALLOC_LIMIT
    torch.cuda.synchronize()
    assert bool((y == 7).all())


def test_noalloc_rowsum_replays_from_a_captured_graph(H):
    """What the entry point is for: recorded into a HIP graph (after a first eager call on the
    device, which looks the scratch array's address up) and replayed.  Every replay, with new
    inputs written eagerly between the replays, gives what the ordinary entry point gives on
    the same inputs: exactly, on small integers."""
    import torch
    m, n = 12, 3 * 8192 + 64                # split form: 12 rows x 4 chunks, the last one short
    gen = torch.Generator(device="cuda").manual_seed(11)

    def ints(shape):
        return torch.randint(-4, 5, shape, generator=gen, device="cuda", dtype=torch.int32).float()

    x, bias = ints((m, n)), ints((n,))
    y = torch.empty((m,), dtype=torch.float32, device="cuda")
    y_plain = torch.empty_like(y)
    tiling = H.pack_tiling(m, n)
    H.prepare(NOALLOC, [x.data_ptr(), bias.data_ptr(), y.data_ptr(), 0], tiling)()    # the warm first call
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        H.prepare(NOALLOC, [x.data_ptr(), bias.data_ptr(), y.data_ptr(), 0], tiling)()   # prepared inside: the capturing stream
    plain = H.prepare(PLAIN, [x.data_ptr(), bias.data_ptr(), y_plain.data_ptr(), 0], tiling)
    for replay in range(4):
        x.copy_(ints((m, n)))
        bias.copy_(ints((n,)))
        plain()
        y.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, y_plain), replay
        assert torch.equal(y.double(), x.double().sum(1) + bias.double().sum()), replay
