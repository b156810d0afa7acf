"""Parity of the HIP fused kernels (called through the C ABI) with the CPU
oracle on the same seeded inputs.  Needs an MI355X: run with -m gpu.

Bars: bit-exact for the f32 add/mul chain, the f16 transpose chain and the
gather; <= 1e-5 relative (with an absolute floor of 1e-7 * sum|terms|, the
scale of one rounding of the row's terms) for the f32 row sum; <= 1e-2 relative (atol 1e-5)
for the bf16 matmul epilogue.
"""
import numpy as np
import pytest

from oracle import afir_oracle as O
from oracle import c_oracle as C

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


@pytest.fixture(scope="module")
def H(pkg):
    from ascend_mlir_amd import hip_kernels
    hip_kernels.load()          # raises if the library is not built
    assert torch.cuda.is_available(), "no GPU visible"
    return hip_kernels


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def dev_bf16(bits):
    return torch.from_numpy(np.ascontiguousarray(bits).view(np.int16)).cuda().view(torch.bfloat16)


def host_bf16(t):
    return t.view(torch.int16).cpu().numpy().view(np.uint16)


# ---------------------------------------------------------------- C1 --------

@pytest.mark.parametrize("shape", [(4, 4), (1, 1), (257, 129), (1024, 1024), (3, 100003)])
def test_c1_small_bit_exact(H, shape):
    a, b = O.gen_c1(shape)
    out = H.fused_add_mul(dev(a), dev(b)).cpu().numpy()
    assert out.tobytes() == O.golden_c1(a, b).tobytes()
    assert out.tobytes() == C.add_mul_f32(a, b).tobytes()


def test_c1_full_size_bit_exact(H):
    a, b = O.gen_c1()
    out = H.fused_add_mul(dev(a), dev(b)).cpu().numpy()
    assert out.tobytes() == O.golden_c1(a, b).tobytes()


# From 16 MiB of output up to 128 MiB the whole 32 KiB blocks of the chain take the kernel that
# separates the chip's reads from its writes in time (two launches above 64 MiB); what is left
# over takes the other kernels.  AFIR_HIP_PHASED=0 keeps a launch off it.
@pytest.mark.parametrize("shape", [(2048, 2049), (3001, 2999), (6000, 4096), (9000, 4096),
                                   # at the limits: 512 blocks (the fewest), one row less, 4096 blocks, half a block more
                                   (1024, 4096), (1023, 4096), (8192, 4096), (8193, 4096)])
def test_c1_phased_route_bit_exact(H, shape, monkeypatch):
    a, b = O.gen_c1(shape)
    a.ravel()[:8] = [0.0, -0.0, np.inf, -np.inf, np.nan, 1e-45, 3e38, 1.0]
    b.ravel()[:8] = [0.0, 0.0, 1.0, np.inf, 1.0, 1e-45, 3e38, -1.0]
    a.ravel()[-3:] = [np.nan, -0.0, 3e38]
    with np.errstate(all="ignore"):
        want = O.golden_c1(a, b)
    ok = ~np.isnan(want)
    for phased in ("1", "0"):
        monkeypatch.setenv("AFIR_HIP_PHASED", phased)
        out = H.fused_add_mul(dev(a), dev(b)).cpu().numpy()
        assert np.array_equal(np.isnan(out), np.isnan(want))
        assert out[ok].tobytes() == want[ok].tobytes()


def test_c1_empty_unaligned_and_blockdim(H):
    e = torch.empty((0, 16), dtype=torch.float32, device="cuda")
    assert H.fused_add_mul(e, e).shape == (0, 16)
    a, b = O.gen_c1((1, 4099))
    da, db = dev(np.concatenate([[0], a.ravel()]).astype(np.float32)), \
        dev(np.concatenate([[0], b.ravel()]).astype(np.float32))
    ua, ub = da[1:].view(1, -1), db[1:].view(1, -1)       # 4-byte aligned only
    out = H.fused_add_mul(ua, ub).cpu().numpy()
    assert out.tobytes() == O.golden_c1(a, b).tobytes()
    a, b = O.gen_c1((512, 1000))
    for bd in (1, 7, 40):                                   # reference-style block_dim
        out = H.fused_add_mul(dev(a), dev(b), block_dim=bd).cpu().numpy()
        assert out.tobytes() == O.golden_c1(a, b).tobytes()


def test_c1_special_values(H):
    a = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 1e-45, 3e38, 1.0], np.float32)
    b = np.array([0.0, 0.0, 1.0, np.inf, 1.0, 1e-45, 3e38, -1.0], np.float32)
    with np.errstate(all="ignore"):
        want = O.golden_c1(a, b)
    out = H.fused_add_mul(dev(a.reshape(1, -1)), dev(b.reshape(1, -1))).cpu().numpy().ravel()
    assert np.array_equal(np.isnan(out), np.isnan(want))
    ok = ~np.isnan(want)
    assert out[ok].tobytes() == want[ok].tobytes()       # denormals are kept


# ---------------------------------------------------------------- C2 --------

def _check_rowsum(x, bias, y):
    want = O.golden_c2(x, bias)
    scale = np.abs(x.astype(np.float64) + bias.astype(np.float64)).sum(axis=1)
    err = np.abs(y.astype(np.float64) - want.astype(np.float64))
    tol = 1e-5 * np.abs(want.astype(np.float64)) + 1e-7 * scale
    assert np.all(err <= tol), (err.max(), (err / np.maximum(tol, 1e-300)).max())
    # and against exact arithmetic: well inside f32 accumulation error
    exact = x.astype(np.float64).sum(axis=1) + bias.astype(np.float64).sum()
    assert np.all(np.abs(y - exact) <= 2e-6 * scale + 1e-30)


@pytest.mark.parametrize("m,n", [(1, 4), (7, 5), (33, 4096), (64, 512), (5, 1000),
                                 (130, 1028), (3, 8192), (2, 100000),
                                 # short rows and few long rows: the family's compiled region kernels
                                 (5000, 100), (3000, 8), (2, 8 * 4096), (70, 24 * 4096), (1500, 2044)])
def test_c2_small(H, m, n):
    x, bias = O.gen_c2(m, n)
    y = H.broadcast_add_reducesum(dev(x), dev(bias)).cpu().numpy()
    _check_rowsum(x, bias, y)


def test_c2_full_size(H):
    x, bias = O.gen_c2()
    y = H.broadcast_add_reducesum(dev(x), dev(bias)).cpu().numpy()
    _check_rowsum(x, bias, y)


def test_c2_exact_integer_rows_and_blockdim(H):
    ones = np.ones((16, 4096), np.float32)
    z = np.zeros(4096, np.float32)
    y = H.broadcast_add_reducesum(dev(ones), dev(z)).cpu().numpy()
    assert np.array_equal(y, np.full(16, 4096, np.float32))
    onehot = np.zeros((4, 128), np.float32)
    onehot[np.arange(4), [0, 5, 77, 127]] = 3.0
    y = H.broadcast_add_reducesum(dev(onehot), dev(np.ones(128, np.float32))).cpu().numpy()
    assert np.array_equal(y, np.full(4, 131, np.float32))
    x, bias = O.gen_c2(100, 640)
    for bd in (1, 40):
        y = H.broadcast_add_reducesum(dev(x), dev(bias), block_dim=bd).cpu().numpy()
        _check_rowsum(x, bias, y)
    e = torch.empty((0, 8), dtype=torch.float32, device="cuda")
    assert H.broadcast_add_reducesum(e, dev(z[:8])).shape == (0,)
    # zero columns: every row sums to 0
    y = H.broadcast_add_reducesum(torch.empty((3, 0), dtype=torch.float32, device="cuda"),
                                  torch.empty((0,), dtype=torch.float32, device="cuda"))
    assert np.array_equal(y.cpu().numpy(), np.zeros(3, np.float32))


# ---------------------------------------------------------------- C3 --------

@pytest.mark.parametrize("b,m,n", [(2, 3, 5), (1, 128, 128), (3, 256, 128), (2, 128, 384),
                                   (3, 70, 36), (1, 1, 1), (2, 129, 128), (1, 33, 250),
                                   # multiples of 8 that are not whole tiles: the family's compiled region kernels
                                   (2, 72, 136), (3, 1024, 520), (1, 200, 64), (2, 64, 72)])
def test_c3_small_bit_exact(H, b, m, n):
    x, c = O.gen_c3(b, m, n)
    out = H.relu_broadcast_add_transpose(dev(x), dev(c)).cpu().numpy()
    assert out.shape == (b, n, m)
    assert out.tobytes() == O.golden_c3(x, c).tobytes()
    assert out.tobytes() == C.relu_bcast_add_transpose_f16(x, c).tobytes()


def test_c3_full_size_bit_exact(H):
    x, c = O.gen_c3()
    out = H.relu_broadcast_add_transpose(dev(x), dev(c)).cpu().numpy()
    assert out.tobytes() == O.golden_c3(x, c).tobytes()


def test_c3_involution_and_blockdim(H):
    x, _ = O.gen_c3(4, 256, 384)
    pos = np.abs(x)
    z1 = dev(np.zeros(384, np.float16))
    z2 = dev(np.zeros(256, np.float16))
    once = H.relu_broadcast_add_transpose(dev(pos), z1)
    twice = H.relu_broadcast_add_transpose(once, z2).cpu().numpy()
    assert twice.tobytes() == pos.tobytes()
    x, c = O.gen_c3(2, 256, 256)
    for bd in (1, 5):
        out = H.relu_broadcast_add_transpose(dev(x), dev(c), block_dim=bd).cpu().numpy()
        assert out.tobytes() == O.golden_c3(x, c).tobytes()
    e = torch.empty((0, 4, 4), dtype=torch.float16, device="cuda")
    assert H.relu_broadcast_add_transpose(e, dev(np.zeros(4, np.float16))).shape == (0, 4, 4)


def test_c3_special_values(H):
    x = np.zeros((1, 128, 128), np.float16)
    x[0, 0, :8] = [np.nan, -np.inf, np.inf, -0.0, 6e-8, -6e-8, 65504, -65504]
    c = np.zeros(128, np.float16)
    c[3] = -0.0
    with np.errstate(all="ignore"):
        want = O.golden_c3(x, c)
    out = H.relu_broadcast_add_transpose(dev(x), dev(c)).cpu().numpy()
    assert np.array_equal(np.isnan(out), np.isnan(want))
    ok = ~np.isnan(want)
    assert out[ok].tobytes() == want[ok].tobytes()


# Shapes of whole 64 x 256 tile groups from 24 MiB up take the kernel that separates the chip's
# reads from its writes in time (up to 128 MiB, in launches of at most 64 MiB); AFIR_HIP_PHASED=0
# keeps a launch on the other kernel.
@pytest.mark.parametrize("b,m,n", [(12, 1024, 1024), (3, 4096, 1024), (40, 512, 768), (64, 512, 1024),
                                   (81, 1024, 512), (130, 1024, 512),      # 41 + 40 batches; past two launches' worth
                                   # at the limits: 767 tile groups (one too few), 4096 (two full launches), 4128
                                   (13, 3776, 256), (128, 1024, 512), (129, 1024, 512)])
def test_c3_phased_route_bit_exact(H, b, m, n, monkeypatch):
    x, c = O.gen_c3(b, m, n)
    x[0, 0, :8] = [np.nan, -np.inf, np.inf, -0.0, 6e-8, -6e-8, 65504, -65504]
    x[-1, -1, -4:] = [np.nan, -0.0, 65504, -1.0]
    c[3] = -0.0
    with np.errstate(all="ignore"):
        want = O.golden_c3(x, c)
    ok = ~np.isnan(want)
    for phased in ("1", "0"):
        monkeypatch.setenv("AFIR_HIP_PHASED", phased)
        out = H.relu_broadcast_add_transpose(dev(x), dev(c)).cpu().numpy()
        assert np.array_equal(np.isnan(out), np.isnan(want))
        assert out[ok].tobytes() == want[ok].tobytes()


# ---------------------------------------------------------------- C4 --------

@pytest.mark.parametrize("rows,dim,nidx", [(512, 64, 256), (1000, 1024, 513), (100, 136, 77),
                                           (64, 8, 5), (300, 2048, 40), (50, 100, 33),
                                           (10, 1, 7), (128, 1536, 19),
                                           # rows of fewer than 256 halves: the family's compiled region kernels
                                           (4096, 64, 30000), (777, 248, 1001), (9, 16, 100000)])
def test_c4_small_bit_exact(H, rows, dim, nidx):
    table, idx, scale, shift = O.gen_c4(rows, dim, nidx)
    idx[:3] = [0, rows - 1, rows - 1]
    out = H.gather_scale_shift(dev(table), dev(idx), dev(scale), dev(shift)).cpu().numpy()
    assert out.tobytes() == O.golden_c4(table, idx, scale, shift).tobytes()
    assert out.tobytes() == C.gather_scale_shift_f16(table, idx, scale, shift).tobytes()


def test_c4_identity_rows_are_byte_identical(H):
    table, idx, _, _ = O.gen_c4(4096, 1024, 2048)
    one = np.ones(1024, np.float16)
    zero = np.zeros(1024, np.float16)
    out = H.gather_scale_shift(dev(table), dev(idx), dev(one), dev(zero)).cpu().numpy()
    assert out.tobytes() == table[idx].tobytes()


def test_c4_full_size_bit_exact(H):
    table, idx, scale, shift = O.gen_c4()
    idx[:4] = [0, 131071, 131071, 0]
    out = H.gather_scale_shift(dev(table), dev(idx), dev(scale), dev(shift)).cpu().numpy()
    assert out.tobytes() == O.golden_c4(table, idx, scale, shift).tobytes()


def test_c4_out_of_range_index_is_flagged_not_read(H):
    table, idx, scale, shift = O.gen_c4(64, 128, 16)
    idx[5] = 64
    idx[9] = -1
    ws = torch.zeros(2, dtype=torch.int32, device="cuda")
    out = H.gather_scale_shift(dev(table), dev(idx), dev(scale), dev(shift),
                               workspace=ws).cpu().numpy()
    assert int(ws[0].item()) != 0
    assert np.isnan(out[5]).all() and np.isnan(out[9]).all()
    good = np.ones(16, bool)
    good[[5, 9]] = False
    idx2 = idx.copy()
    idx2[[5, 9]] = 0
    want = O.golden_c4(table, idx2, scale, shift)
    assert out[good].tobytes() == want[good].tobytes()
    ws.zero_()
    H.gather_scale_shift(dev(table), dev(idx2), dev(scale), dev(shift), workspace=ws)
    assert int(ws[0].item()) == 0
    e = torch.empty((0,), dtype=torch.int32, device="cuda")
    assert H.gather_scale_shift(dev(table), e, dev(scale), dev(shift)).shape == (0, 128)


def test_c4_blockdim(H):
    table, idx, scale, shift = O.gen_c4(777, 1024, 1000)
    want = O.golden_c4(table, idx, scale, shift)
    for bd in (1, 3, 40):
        out = H.gather_scale_shift(dev(table), dev(idx), dev(scale), dev(shift),
                                   block_dim=bd).cpu().numpy()
        assert out.tobytes() == want.tobytes()


# Gathers whose rows are 32 * 2^k halves take the kernel that separates the chip's reads from its
# writes in time (whole blocks of rows, up to 128 MiB in launches of at most 64 MiB; rows left
# over take the other kernel in a launch of their own).  AFIR_HIP_PHASED=0 keeps a launch off it.
@pytest.mark.parametrize("dim,nidx", [(1024, 16), (1024, 17), (1024, 513), (1024, 4099), (256, 64), (256, 1000),
                                      (2048, 8), (2048, 77), (8192, 2), (8192, 31), (32, 512), (32, 70001),
                                      (1024, 40000), (1024, 70003),      # two launches; past two launches' worth
                                      (1024, 65536), (1024, 65552)])     # at the limit: two full launches, one block more
def test_c4_phased_route_bit_exact(H, dim, nidx, monkeypatch):
    rows = 3000
    table, idx, scale, shift = O.gen_c4(rows, dim, nidx)
    idx[:2] = [rows - 1, 0]
    idx[-1] = rows - 1
    want = O.golden_c4(table, idx, scale, shift)
    out = H.gather_scale_shift(dev(table), dev(idx), dev(scale), dev(shift)).cpu().numpy()
    assert out.tobytes() == want.tobytes()
    monkeypatch.setenv("AFIR_HIP_PHASED", "0")
    out = H.gather_scale_shift(dev(table), dev(idx), dev(scale), dev(shift)).cpu().numpy()
    assert out.tobytes() == want.tobytes()


def test_c4_phased_launch_needs_every_lane_resident(H, monkeypatch):
    """Rows of 8192 halves park 32 KiB of scale / shift per workgroup in LDS: five workgroups of
    256 lanes fit a compute unit, not the eight that put a whole launch in flight at once (asked
    of the runtime: the occupancy of the kernel with that much LDS), so such gathers run as four
    workgroups of 512 lanes per compute unit; a row count whose workgroups would leave many
    compute units idle at the end keeps to the grouped kernel.  Rows of 4096 halves fit as 256
    lanes.  The hold constants are read from the environment at every launch: a hold far too
    short or too long changes the timing only."""
    table, idx, scale, shift = O.gen_c4(5000, 8192, 4096)
    out = H.gather_scale_shift(dev(table), dev(idx), dev(scale), dev(shift)).cpu().numpy()
    assert out.tobytes() == O.golden_c4(table, idx, scale, shift).tobytes()
    note = H.last_launch()
    assert note["kernel"] == "gather_scale_shift_f16_phased" and note["workgroups"] == 1024 and note["threads"] == 512
    table, idx, scale, shift = O.gen_c4(5000, 8192, 2560)      # 640 workgroups: 2.5 per compute unit
    out = H.gather_scale_shift(dev(table), dev(idx), dev(scale), dev(shift)).cpu().numpy()
    assert out.tobytes() == O.golden_c4(table, idx, scale, shift).tobytes()
    assert H.last_launch()["kernel"] == "gather_scale_shift_f16_grouped"
    table, idx, scale, shift = O.gen_c4(5000, 4096, 8192)
    want = O.golden_c4(table, idx, scale, shift)
    args = (dev(table), dev(idx), dev(scale), dev(shift))
    out = H.gather_scale_shift(*args).cpu().numpy()
    note = H.last_launch()
    assert out.tobytes() == want.tobytes()
    assert note["kernel"] == "gather_scale_shift_f16_phased" and note["workgroups"] == 2048 and note["threads"] == 256
    for gbs, base in (("100000", "0"), ("1000", "5000")):
        monkeypatch.setenv("AFIR_GATHER_PHASE_GBS", gbs)
        monkeypatch.setenv("AFIR_GATHER_PHASE_BASE_NS", base)
        assert H.gather_scale_shift(*args).cpu().numpy().tobytes() == want.tobytes()


def test_c4_phased_route_flags_bad_indices(H):
    table, idx, scale, shift = O.gen_c4(500, 1024, 100)
    idx[[3, 40, 99]] = [500, -7, 1 << 30]       # rows 3 and 40 in whole blocks, 99 among the rows left over
    ws = torch.zeros(2, dtype=torch.int32, device="cuda")
    out = H.gather_scale_shift(dev(table), dev(idx), dev(scale), dev(shift), workspace=ws).cpu().numpy()
    assert int(ws[0].item()) != 0
    good = np.ones(100, bool)
    good[[3, 40, 99]] = False
    assert np.isnan(out[~good]).all()
    idx2 = idx.copy()
    idx2[~good] = 0
    assert out[good].tobytes() == O.golden_c4(table, idx2, scale, shift)[good].tobytes()


# ---------------------------------------------------------------- C5 --------

C5_ATOL, C5_RTOL = 1e-5, 1e-2


def _check_c5(got_bits, want_bits):
    r = O.compare_outputs([(got_bits, "bf16")], [(want_bits, "bf16")], C5_ATOL, C5_RTOL)
    assert r["passed"], r
    # the comparator's `diff > tol` is false for NaN: count those separately
    assert O.nonfinite_mismatches(got_bits, want_bits, "bf16") == 0
    assert (got_bits == want_bits).mean() > 0.97


@pytest.mark.parametrize("m,k,n", [(256, 256, 256), (512, 128, 768), (128, 64, 128),
                                   (384, 192, 128), (48, 1024, 80), (1, 1, 1), (17, 33, 65),
                                   (256, 100, 256),
                                   # K and N multiples of 8, nothing else aligned: the bounds-checked MFMA kernel
                                   (1, 8, 8), (130, 72, 136), (1000, 1000, 1000), (257, 8, 520), (300, 1096, 24),
                                   # odd extents: the same kernel with element accesses
                                   (257, 129, 513), (300, 1001, 517), (129, 1, 127), (2048, 3, 9)])
def test_c5_small(H, m, k, n):
    a, b, bias = O.gen_c5(m, k, n)
    out = H.matmul_add_leakyrelu(dev_bf16(a), dev_bf16(b), dev_bf16(bias), 0.01)
    _check_c5(host_bf16(out), O.golden_c5(a, b, bias, 0.01))


def test_c5_integer_known_answer_exact(H):
    # the reference's trick: small integers make f32 accumulation exact, so any
    # summation order must give the same bits
    r = np.random.default_rng(42)
    for (m, k, n) in [(128, 256, 128), (256, 512, 512)]:
        A = r.integers(-10, 10, (m, k)).astype(np.float32)
        B = r.integers(-10, 10, (k, n)).astype(np.float32)
        bias = r.integers(1, 10, (n,)).astype(np.float32)
        bits = [O.f32_to_bf16_bits(v) for v in (A, B, bias)]
        out = H.matmul_add_leakyrelu(dev_bf16(bits[0]), dev_bf16(bits[1]), dev_bf16(bits[2]), 0.01)
        assert np.array_equal(host_bf16(out), O.golden_c5(*bits, 0.01))


@pytest.mark.parametrize("ty", ["bf16", "f16"])
def test_c5_ragged_shapes_integer_known_answer_exact(H, ty):
    """Shapes that are not multiples of the tiles, on small integers (every product and
    partial sum exact in float32): the bounds-checked MFMA kernel must reproduce
    leakyrelu(A @ B + bias) exactly and leave the rows next to the output alone."""
    import os
    import subprocess
    from oracle import region_oracle as RO
    from tests import mlir_cases as MC
    # (the last shape: whole 256 x 256 tiles on the direct-to-LDS kernel, the 37 rows left over on
    # the bounds-checked one, in two launches)
    for (m, k, n) in ((1000, 1000, 1000), (129, 136, 264), (5, 64, 8), (301, 1001, 517), (131, 7, 129), (2048 + 37, 512, 4096)):
        rng = np.random.default_rng(m + k)
        a = rng.integers(-3, 4, (m, k)).astype(np.float32)
        b = rng.integers(-3, 4, (k, n)).astype(np.float32)
        bias = rng.integers(-8, 9, (n,)).astype(np.float32)
        v = a @ b + bias[None, :]
        assert np.abs(v).max() < 2 ** 24
        if ty == "bf16":
            bits = [O.f32_to_bf16_bits(x) for x in (a, b, bias)]
            guard = torch.full((m + 2, n), 7.0, dtype=torch.bfloat16, device="cuda")
            out = H.matmul_add_leakyrelu(dev_bf16(bits[0]), dev_bf16(bits[1]), dev_bf16(bits[2]), 0.25, out=guard[1:m + 1])
            torch.cuda.synchronize()
            assert np.array_equal(host_bf16(out), O.golden_c5(*bits, 0.25)), (m, k, n)
            assert bool((guard[0] == 7).all()) and bool((guard[m + 1] == 7).all())
        else:
            tr = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "ascend-mlir_amd", "bin",
                              "afir-translate")
            text = subprocess.run([tr, "-mlir-to-hip", "-"], input=MC.MATMUL_BIAS_LEAKY_F16, capture_output=True,
                                  text=True, check=True).stdout
            r = H.Region(text)
            ins = [a.astype(np.float16), b.astype(np.float16), bias, np.zeros((m, n), np.float32)]
            got = r(*[dev(x) for x in ins], out_shape=(m, n)).cpu().numpy()
            r.close()
            assert got.tobytes() == RO.evaluate(text, ins).tobytes(), (m, k, n)
            assert np.array_equal(got, np.maximum(v, v * np.float32(0.001)))


def test_c5_f16_direct_to_lds_kernel_integer_known_answer_exact(H):
    """f16 inputs, float32 bias and output (the reference example's types) at shapes of whole
    256 x 256 tiles, enough of them for the direct-to-LDS kernel: on small integers every
    product and partial sum is exact in float32, so the result must be leakyrelu(A @ B + bias)
    to the bit, which also pins the permutation of the float32 epilogue's staging."""
    import os
    import subprocess
    from tests import mlir_cases as MC
    tr = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "ascend-mlir_amd", "bin",
                      "afir-translate")
    text = subprocess.run([tr, "-mlir-to-hip", "-"], input=MC.MATMUL_BIAS_LEAKY_F16, capture_output=True,
                          text=True, check=True).stdout
    r = H.Region(text)
    for (m, k, n) in ((4096, 512, 2048), (2048, 320, 4096), (2304, 256, 3840)):
        rng = np.random.default_rng(m + k)
        a = rng.integers(-3, 4, (m, k)).astype(np.float32)
        b = rng.integers(-3, 4, (k, n)).astype(np.float32)
        bias = rng.integers(-8, 9, (n,)).astype(np.float32)
        v = a @ b + bias[None, :]
        assert np.abs(v).max() < 2 ** 24
        guard = torch.full((m + 2, n), 7.0, dtype=torch.float32, device="cuda")
        ins = [dev(a.astype(np.float16)), dev(b.astype(np.float16)), dev(bias), torch.zeros((m, n), device="cuda")]
        got = guard[1:m + 1]
        dims = [d for t in ins for d in t.shape] + [m, n]
        assert r.launch_raw([t.data_ptr() for t in ins] + [got.data_ptr()], H.pack_tiling(*dims)) == 0
        torch.cuda.synchronize()
        assert np.array_equal(got.cpu().numpy(), np.maximum(v, v * np.float32(0.001))), (m, k, n)
        assert bool((guard[0] == 7).all()) and bool((guard[m + 1] == 7).all())
    r.close()


def test_c5_identity_and_alpha(H):
    n = 256
    eye = O.f32_to_bf16_bits(np.eye(n, dtype=np.float32))
    a, _, _ = O.gen_c5(n, n, n)
    zero = np.zeros(n, np.uint16)
    out = H.matmul_add_leakyrelu(dev_bf16(a), dev_bf16(eye), dev_bf16(zero), 1.0)
    assert np.array_equal(host_bf16(out), a)                 # alpha=1: identity
    out = H.matmul_add_leakyrelu(dev_bf16(a), dev_bf16(eye), dev_bf16(zero), 0.0)
    want = O.f32_to_bf16_bits(np.maximum(O.bf16_bits_to_f32(a), 0))
    got = host_bf16(out)
    assert np.array_equal(O.bf16_bits_to_f32(got), O.bf16_bits_to_f32(want))   # relu (-0 == 0)


def test_c5_full_size(H):
    a, b, bias = O.gen_c5()
    out = H.matmul_add_leakyrelu(dev_bf16(a), dev_bf16(b), dev_bf16(bias), 0.01)
    got = host_bf16(out)
    want = O.golden_c5(a, b, bias, 0.01)
    _check_c5(got, want)


def test_c5_empty_and_blockdim(H):
    a, b, bias = O.gen_c5(512, 128, 512)
    want = O.golden_c5(a, b, bias, 0.01)
    for bd in (1, 3):
        out = H.matmul_add_leakyrelu(dev_bf16(a), dev_bf16(b), dev_bf16(bias), 0.01, block_dim=bd)
        _check_c5(host_bf16(out), want)
    e = torch.empty((0, 128), dtype=torch.bfloat16, device="cuda")
    out = H.matmul_add_leakyrelu(e, dev_bf16(b), dev_bf16(bias), 0.01)
    assert out.shape == (0, 512)


# ------------------------------------------------------- dispatch by name ----

def test_tensors_of_more_than_2_to_31_elements(H):
    """The hand-tuned kernels on tensors whose element positions do not fit 32 bits.  The
    inputs are small integers made on the GPU (too large for the numpy oracle to be quick);
    the expected values come from torch's own elementwise, sum, transpose and indexing
    kernels, slice by slice, and every result is exact."""
    gen = torch.Generator(device="cuda").manual_seed(9)

    def ints(shape, dtype, lo=-3, hi=4):
        t = torch.empty(shape, dtype=dtype, device="cuda")
        flat = t.view(-1)
        step = 1 << 28
        for i0 in range(0, flat.numel(), step):
            part = flat[i0:i0 + step]
            part.copy_(torch.randint(lo, hi, part.shape, generator=gen, device="cuda", dtype=torch.int8))
        return t

    rows, n = 32776, 65536                     # 2^31 + 2^19 elements
    # C1: (a + b) * b, f32
    a, b = ints((rows, n), torch.float32), ints((rows, n), torch.float32)
    out = H.fused_add_mul(a, b)
    for r0 in range(0, rows, 4096):
        assert torch.equal(out[r0:r0 + 4096], (a[r0:r0 + 4096] + b[r0:r0 + 4096]) * b[r0:r0 + 4096]), r0
    del b, out
    # C2: row sums of x + bias, f32 (integers: exact in any order)
    bias = ints((n,), torch.float32)
    y = H.broadcast_add_reducesum(a, bias)
    want = torch.cat([(a[r0:r0 + 2048] + bias).sum(dim=1) for r0 in range(0, rows, 2048)])
    assert torch.equal(y, want)
    del a, y, want
    # C3: out[b, j, i] = relu(x[b, i, j]) + c[j], f16
    x = ints((33, 8192, 8192), torch.float16)
    c = ints((8192,), torch.float16)
    out = H.relu_broadcast_add_transpose(x, c)
    for k in range(33):
        assert torch.equal(out[k], (torch.relu(x[k]) + c).t()), k
    del x, out
    # C4: rows of a table of 2^31 + 2^21 elements, the last rows among them
    table = ints((2099200, 1024), torch.float16)
    idx = torch.randint(0, 2099200, (4096,), generator=gen, device="cuda", dtype=torch.int32)
    idx[:4] = torch.tensor([2099199, 2097152, 0, 2099198], dtype=torch.int32)
    scale, shift = ints((1024,), torch.float16, 1, 4), ints((1024,), torch.float16)
    got = H.gather_scale_shift(table, idx, scale, shift)
    assert torch.equal(got, table[idx.long()] * scale + shift)


def test_launch_by_name_and_errors(H):
    import ctypes
    L = H.load()
    a, b = O.gen_c1((64, 64))
    da, db = dev(a), dev(b)
    out = torch.empty_like(da)
    args = (ctypes.c_void_p * 3)(da.data_ptr(), db.data_ptr(), out.data_ptr())
    til = H.pack_tiling(64, 64)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    rc = L.afir_hip_launch(b"fused_add_mul", 0, stream, 3, args, None, til, len(til))
    assert rc == 0
    torch.cuda.synchronize()
    assert out.cpu().numpy().tobytes() == O.golden_c1(a, b).tobytes()
    assert L.afir_hip_launch(b"no_such_kernel", 0, stream, 3, args, None, til, len(til)) == 3
    assert b"no_such_kernel" in L.afir_hip_last_error()
    assert L.afir_hip_launch(b"fused_add_mul", 0, stream, 2, args, None, til, len(til)) == 1
    assert L.afir_hip_launch(b"fused_add_mul", 0, stream, 3, args, None, til, 8) == 1
    assert b"tiling" in L.afir_hip_last_error()
    bad = H.pack_tiling(-1, 64)
    assert L.afir_hip_launch(b"fused_add_mul", 0, stream, 3, args, None, bad, len(bad)) == 1
