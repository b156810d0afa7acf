"""Fused-region programs against the region oracle, on the interpreter kernel
(chain and stack evaluators) and on kernels compiled for each program: the
reference's example graphs at their own shapes, the benchmark configurations as
programs, ragged / unaligned shapes, and seeded random op chains.  Needs a GPU
(and hipcc for the compiled mode)."""
import numpy as np
import pytest

from oracle import afir_oracle as O
from oracle import region_oracle as RO
from tests import region_cases as RC

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def H(pkg):
    import torch
    from ascend_mlir_amd import hip_kernels
    hip_kernels.load()
    assert torch.cuda.is_available()
    return hip_kernels


def _dev(x, t):
    import torch
    if t == "bf16":
        return torch.from_numpy(x.view(np.int16)).cuda().view(torch.bfloat16)
    return torch.from_numpy(np.ascontiguousarray(x)).cuda()


def _host(t, ty):
    import torch
    if ty == "bf16":
        return t.view(torch.int16).cpu().numpy().view(np.uint16)
    return t.cpu().numpy()


MODE = {"compiled": False, "cache": None}


@pytest.fixture(params=["chain", "stack", "compiled"], autouse=True)
def evaluator(request, monkeypatch, tmp_path_factory):
    """Every test runs three times: expressions that are chains on the linear
    form of the interpreter, everything on its stack form, and everything on
    kernels emitted and compiled for the program."""
    monkeypatch.setenv("AFIR_HIP_REGION_GENERIC", "1")
    if request.param == "stack":
        monkeypatch.setenv("AFIR_HIP_REGION_STACK", "1")
    MODE["compiled"] = request.param == "compiled"
    if MODE["cache"] is None:
        MODE["cache"] = str(tmp_path_factory.mktemp("region_cache"))
    yield request.param
    MODE["compiled"] = False


def region(H, text):
    r = H.Region(text)
    if MODE["compiled"]:
        r.compile(cache_dir=MODE["cache"])
        assert r.kernel == "fused_region_compiled"
    return r


def run(H, text, inputs, out_shape, workspace=None, block_dim=0):
    r = region(H, text)
    dev = [_dev(x, r.arg_types[i]) for i, x in enumerate(inputs)]
    out = r(*dev, out_shape=out_shape, workspace=workspace, block_dim=block_dim)
    res = _host(out, r.arg_types[-1])
    r.close()
    return res


@pytest.mark.parametrize("name", sorted(RC.EXACT_CASES))
def test_reference_examples_and_configs_bit_exact(H, name):
    text, inputs, want = RC.EXACT_CASES[name]()
    got = run(H, text, inputs, want.shape)
    assert got.tobytes() == want.tobytes()


@pytest.mark.parametrize("name", sorted(RC.REDUCE_CASES))
def test_reductions_within_tolerance(H, name):
    text, inputs, want = RC.REDUCE_CASES[name]()
    got = run(H, text, inputs, want.shape).astype(np.float64)
    terms = (inputs[0].astype(np.float64)[:, None] + inputs[1].astype(np.float64)
             if inputs[0].ndim == 1 else inputs[0].astype(np.float64) + inputs[1].astype(np.float64))
    scale = np.abs(terms).sum(axis=1)
    ulp = 2.0 ** -10 if want.dtype == np.float16 else 0.0      # one f16 rounding of the result
    tol = 1e-5 * np.abs(want.astype(np.float64)) + 1e-6 * scale + ulp * np.abs(want.astype(np.float64))
    assert np.all(np.abs(got - want.astype(np.float64)) <= tol)


@pytest.mark.parametrize("ty,n", [("f32", 1024), ("f32", 2048), ("f32", 4096), ("f16", 2048), ("f16", 4096),
                                  ("f16", 8192), ("f32", 3072), ("f16", 1024)])
@pytest.mark.parametrize("rows", [1, 5, 1100])
def test_row_sums_of_workgroup_sized_rows(H, ty, n, rows):
    """Rows of 256 lanes x 4 groups (4096 floats, 8192 halves) take the compiled
    workgroup-per-row kernel; with 1100 rows the grid is held to 7 workgroups, so every
    workgroup fetches rows ahead.  The other lengths stay on the wavefront-per-row
    kernel.  Sums of small integers are exact in
    float32 whatever the order, so the result must equal the oracle's bit for bit; a
    second run with uniform values is held to the tolerance of a reordered sum."""
    dt = np.float32 if ty == "f32" else np.float16
    text = RC.C2_BCAST_ADD_ROWSUM.replace("f32", ty)
    rng = np.random.default_rng(rows * 7 + n)
    x = rng.integers(-4, 5, (rows, n)).astype(dt)
    bias = rng.integers(-4, 5, (n,)).astype(dt)
    want = RO.evaluate(text, [x, bias])
    block_dim = 7 if rows == 1100 else 0
    got = run(H, text, [x, bias], (rows,), block_dim=block_dim)
    assert got.tobytes() == want.tobytes()
    x = rng.uniform(-1, 1, (rows, n)).astype(dt)
    bias = rng.uniform(-1, 1, (n,)).astype(dt)
    want = RO.evaluate(text, [x, bias]).astype(np.float64)
    got = run(H, text, [x, bias], (rows,), block_dim=block_dim).astype(np.float64)
    scale = np.abs(x.astype(np.float64) + bias.astype(np.float64)).sum(axis=1)
    ulp = 2.0 ** -10 if ty == "f16" else 0.0
    assert np.all(np.abs(got - want) <= 1e-5 * np.abs(want) + 1e-6 * scale + ulp * np.abs(want))


@pytest.mark.parametrize("rows,n", [(640, 512), (40, 75), (7, 40), (33, 8192), (5, 65536), (16, 1 << 20), (1000, 16)])
def test_mean_is_the_row_sum_divided_by_the_extent_on_every_reduce_kernel(H, rows, n):
    """reduce sum followed by a division by the extent (the reference's mean example), at shapes
    that take each of the row-sum kernels: lanes sharing short rows, a wavefront per row, a
    workgroup per row, a workgroup walking a long row, split and join.  On small integers the
    sum is exact whatever the order, so the result must equal the oracle's bit for bit; on
    uniform values it is held to one unit in the last place of the f16 result.  (The reference's
    graph converts N to f16, which holds it exactly up to 2048 and overflows to infinity from
    65520 on, and keeps the sums in an f16 tensor, where a row of a million terms overflows as
    well; the longer rows take N as a float32 extent and divide the float32 sum.)"""
    text = RC.MEAN_ROWBIAS if n <= 2048 else RC.MEAN_ROWBIAS.replace("const arg1.1 f16", "const arg1.1").replace("  cast f16\n", "")
    rng = np.random.default_rng(rows + n)
    a = rng.integers(-4, 5, (rows,)).astype(np.float16)
    b = rng.integers(-4, 5, (rows, n)).astype(np.float16)
    want = RO.evaluate(text, [a, b])
    got = run(H, text, [a, b], (rows,))
    assert got.tobytes() == want.tobytes()
    a = rng.uniform(-1, 1, (rows,)).astype(np.float16)
    b = rng.uniform(-1, 1, (rows, n)).astype(np.float16)
    want = RO.evaluate(text, [a, b])
    got = run(H, text, [a, b], (rows,))
    exact = (a.astype(np.float64)[:, None] + b.astype(np.float64)).mean(axis=1)
    ulp = np.maximum(np.abs(exact), 2.0 ** -14) * 2.0 ** -10
    assert np.all(np.abs(got.astype(np.float64) - exact) <= ulp + 1e-5 * np.abs(b.astype(np.float64)).mean(axis=1))
    assert np.all(np.abs(got.astype(np.float64) - want.astype(np.float64)) <= 2 * ulp)


def test_mean_graph_from_mlir_runs_on_every_route(H):
    """MLIR text -> program (extent through index_cast + sitofp) -> kernels."""
    import os
    import subprocess
    from tests import mlir_cases as MC
    tr = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "ascend-mlir_amd", "bin", "afir-translate")
    text = subprocess.run([tr, "-mlir-to-hip", "-"], input=MC.ROW_BIAS_MEAN, capture_output=True, text=True, check=True).stdout
    _, inputs, want = RC.case_mean_rowbias(96, 2048)
    got = run(H, text, inputs, want.shape)
    assert np.abs(got.view(np.int16).astype(int) - want.view(np.int16).astype(int)).max() <= 1


def test_mixed_precision_and_named_op_graphs_from_mlir_run_on_every_route(H):
    """MLIR text with arith.truncf / extf, linalg named ops, unit-dim reshapes and afir.cast
    (tests/mlir_cases.py) -> program -> the interpreter's two evaluators and the compiled
    kernels, bit for bit against the region oracle."""
    import os
    import subprocess
    from tests import mlir_cases as MC
    tr = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "ascend-mlir_amd", "bin", "afir-translate")
    rng = np.random.default_rng(21)
    a = rng.uniform(-3, 3, (33, 520)).astype(np.float32)
    a[0, :6] = [65519.9, 65520.0, 1e6, 6e-8, np.nan, -np.inf]
    b = rng.uniform(-3, 3, (520,)).astype(np.float16)
    text = subprocess.run([tr, "-mlir-to-hip", "-"], input=MC.MIXED_PRECISION_CHAIN, capture_output=True, text=True, check=True).stdout
    with np.errstate(all="ignore"):
        want = RO.evaluate(text, [a, b])
    got = run(H, text, [a, b], a.shape)
    assert got.tobytes() == want.tobytes()
    text = subprocess.run([tr, "-mlir-to-hip", "-"], input=MC.NAMED_OPS_GRAPH, capture_output=True, text=True, check=True).stdout
    x, y, c = (rng.uniform(-2, 2, sh).astype(np.float32) for sh in ((4, 8), (8, 4), (8,)))
    assert run(H, text, [x, y, c], (4, 8)).tobytes() == RO.evaluate(text, [x, y, c]).tobytes()
    text = subprocess.run([tr, "-mlir-to-hip", "-"], input=MC.ELEMENTWISE_KIND_SUB, capture_output=True, text=True, check=True).stdout
    p, q = rng.uniform(-2, 2, (7, 40)).astype(np.float16), rng.uniform(-2, 2, (5, 1, 40)).astype(np.float16)
    init = np.zeros((5, 7, 40), np.float16)
    assert run(H, text, [p, q, init], (5, 7, 40)).tobytes() == RO.evaluate(text, [p, q, init]).tobytes()
    # linalg.reduce over named elementwise ops: a row sum, <= 1e-5 relative
    text = subprocess.run([tr, "-mlir-to-hip", "-"], input=MC.NAMED_REDUCE_GRAPH, capture_output=True, text=True, check=True).stdout
    x, bias = rng.uniform(1, 2, (37, 1000)).astype(np.float32), rng.uniform(0, 1, (1000,)).astype(np.float32)
    want = (1.0 / (x.astype(np.float64) ** 2 + bias.astype(np.float64))).sum(axis=1)
    got = run(H, text, [x, bias], (37,)).astype(np.float64)
    assert np.all(np.abs(got - want) <= 1e-5 * np.abs(want))


@pytest.mark.parametrize("n", [1, 3, 8, 16, 40, 64, 100, 256, 520])
def test_row_sums_of_short_rows(H, n):
    """Rows shorter than a pass of the wavefront: 1, 2, 4 ... 32 lanes share a row and a
    wavefront takes several rows; row counts that leave the last wavefront partly empty."""
    rng = np.random.default_rng(n)
    for ty, dt in (("f32", np.float32), ("f16", np.float16)):
        text = RC.C2_BCAST_ADD_ROWSUM.replace("f32", ty)
        for rows in (1, 7, 1000):
            x = rng.integers(-4, 5, (rows, n)).astype(dt)
            bias = rng.integers(-4, 5, (n,)).astype(dt)
            want = RO.evaluate(text, [x, bias])
            assert run(H, text, [x, bias], (rows,)).tobytes() == want.tobytes(), (ty, rows, n)


@pytest.mark.parametrize("ty,n", [("f32", 8192), ("f32", 3 * 4096), ("f16", 16384), ("f16", 5 * 8192)])
def test_row_sums_of_few_long_rows(H, ty, n):
    """A few rows of several workgroup passes each take the compiled long-row kernel: a
    workgroup per row, pass by pass; with two workgroups for seven rows each workgroup also
    moves on to further rows."""
    dt = np.float32 if ty == "f32" else np.float16
    rng = np.random.default_rng(n)
    text = RC.C2_BCAST_ADD_ROWSUM.replace("f32", ty)
    for rows, block_dim in ((1, 0), (7, 0), (7, 2)):
        x = rng.integers(-2, 3, (rows, n)).astype(dt)
        bias = rng.integers(-2, 3, (n,)).astype(dt)
        want = RO.evaluate(text, [x, bias])
        assert np.isfinite(want.astype(np.float32)).all()
        assert run(H, text, [x, bias], (rows,), block_dim=block_dim).tobytes() == want.tobytes(), (rows, block_dim)
    r = rng.integers(-1, 2, (6,)).astype(dt)                    # an operand that changes with the row
    x = rng.integers(-3, 4, (6, n)).astype(dt)
    text = RC.REDUCE_ROWBIAS.replace("f16", ty)
    want = RO.evaluate(text, [r, x])
    assert np.isfinite(want.astype(np.float32)).all()
    assert run(H, text, [r, x], (6,), block_dim=4).tobytes() == want.tobytes()


@pytest.mark.parametrize("ty,n", [("f32", 8 * 4096), ("f32", 37 * 4096), ("f16", 16 * 8192), ("f16", 1000 * 8192)])
@pytest.mark.parametrize("rows", [1, 3, 64])
def test_row_sums_of_a_handful_of_very_long_rows(H, ty, n, rows):
    """Up to 64 rows of eight or more workgroup passes: the compiled split / join pair
    (several workgroups per row leave partial sums, a wavefront per row adds them).  Small
    integers: exact whatever the order, so equal to the oracle bit for bit; run twice to see
    that nothing is left over in the partial sums."""
    dt = np.float32 if ty == "f32" else np.float16
    if rows * n > 40_000_000:
        pytest.skip("kept small for the numpy oracle")
    rng = np.random.default_rng(n + rows)
    text = RC.REDUCE_ROWBIAS.replace("f16", ty)            # r[d0] + x[d0, d1]
    for _ in range(2):
        r = rng.integers(-1, 2, (rows,)).astype(dt) * dt(2.0 ** -8)       # n of them stay below the f16 range
        x = rng.integers(-2, 3, (rows, n)).astype(dt) * dt(0.25)
        want = RO.evaluate(text, [r, x])
        assert np.isfinite(want.astype(np.float32)).all()
        assert run(H, text, [r, x], (rows,)).tobytes() == want.tobytes()


def test_row_sums_with_a_row_operand_and_rank_3(H):
    """The workgroup-per-row kernels with an operand that changes with the row (fetched
    ahead with the matrix) and over a rank-3 space whose row is (d0, d1)."""
    rng = np.random.default_rng(31)
    text = RC.REDUCE_ROWBIAS                                   # r[d0] + x[d0, d1], f16, n = 8192
    r = rng.integers(-3, 4, (300,)).astype(np.float16)
    x = rng.integers(-3, 4, (300, 8192)).astype(np.float16)
    assert run(H, text, [r, x], (300,), block_dim=11).tobytes() == RO.evaluate(text, [r, x]).tobytes()
    text3 = RC.HEADER + ("arg in f32 3\narg in f32 2\narg out f32 2\nsegment 3\n size arg0.0 arg0.1 arg0.2\n outoff 0\n"
                         " push arg0 d0 d1 d2\n push arg1 d0 d2\n mul\n reduce sum\n store\nend\n")
    a = rng.integers(-3, 4, (7, 50, 4096)).astype(np.float32)
    b = rng.integers(-3, 4, (7, 4096)).astype(np.float32)
    assert run(H, text3, [a, b], (7, 50), block_dim=13).tobytes() == RO.evaluate(text3, [a, b]).tobytes()


@pytest.mark.parametrize("shape", [(1, 1), (3, 5), (7, 8), (5, 9), (64, 1000), (2, 4099), (0, 8), (4, 0)])
def test_ragged_shapes_and_block_dim(H, shape):
    rng = np.random.default_rng(11)
    a = rng.uniform(-2, 2, shape).astype(np.float32)
    b = rng.uniform(-2, 2, shape).astype(np.float32)
    want = RO.evaluate(RC.C1_ADD_MUL, [a, b])
    for bd in (0, 1, 7):
        got = run(H, RC.C1_ADD_MUL, [a, b], shape, block_dim=bd)
        assert got.tobytes() == want.tobytes()


@pytest.mark.parametrize("shape", [(1 << 20,), ((1 << 20) + 13,), (3, 300000), (2, 5, 70001), (1, 9000)])
def test_few_long_rows_are_spread_along_the_row(H, shape):
    """Rank-1 tensors and a few very long rows: more workgroups than rows, each taking
    stretches of the row; whole passes and ragged tails, f16 and f32."""
    rng = np.random.default_rng(len(shape) * 100 + shape[-1] % 97)
    rank = len(shape)
    dims = " ".join(f"d{k}" for k in range(rank))
    size = " ".join(f"arg0.{k}" for k in range(rank))
    for ty, dt in (("f16", np.float16), ("f32", np.float32)):
        text = RC.HEADER + (f"arg in {ty} {rank}\narg in {ty} 1\narg out {ty} {rank}\nsegment {rank}\n size {size}\n outoff 0\n"
                            f" push arg0 {dims}\n push arg1 d{rank - 1}\n mul\n relu\n store\nend\n")
        x = rng.uniform(-2, 2, shape).astype(dt)
        c = rng.uniform(-2, 2, shape[-1:]).astype(dt)
        want = RO.evaluate(text, [x, c])
        got = run(H, text, [x, c], shape)
        assert got.tobytes() == want.tobytes(), (ty, shape)


def test_positions_beyond_32_bits(H):
    """Tensors of more than 2^31 elements take the kernels with 64-bit positions: an
    elementwise region, a row sum and a transposed read over [32776, 65536] halves (4.3 GB
    each).  Too large for the numpy oracle to be quick, so the inputs are made on the GPU
    and the expected values come from torch's own elementwise, sum and transpose kernels."""
    import torch
    rows, n = 32776, 65536
    assert rows * n > 2 ** 31
    gen = torch.Generator(device="cuda").manual_seed(5)
    x = torch.empty((rows, n), dtype=torch.float16, device="cuda")
    for r0 in range(0, rows, 4096):          # filled in pieces: no float32 copy of the whole tensor
        part = x[r0:r0 + 4096]
        part.copy_(torch.randint(-3, 4, part.shape, generator=gen, device="cuda", dtype=torch.int8))
    c = torch.randint(-3, 4, (n,), generator=gen, device="cuda", dtype=torch.int8).to(torch.float16)
    head = RC.HEADER + "arg in f16 2\narg in f16 1\n"
    # relu(x * c): small integers, every product exact
    text = head + "arg out f16 2\nsegment 2\n size arg0.0 arg0.1\n outoff 0\n push arg0 d0 d1\n push arg1 d1\n mul\n relu\n store\nend\n"
    r = region(H, text)
    out = r(x, c, out_shape=(rows, n))
    r.close()
    for r0 in range(0, rows, 4096):
        assert torch.equal(out[r0:r0 + 4096], torch.relu(x[r0:r0 + 4096] * c)), r0
    # the last rows lie beyond element 2^31
    assert (rows - 1) * n > 2 ** 31 and bool((out[-1] == torch.relu(x[-1] * c)).all())
    del out
    # row sums of x * c: integers below 2^24, exact in float32 in any order
    text = head + "arg out f32 1\nsegment 2\n size arg0.0 arg0.1\n outoff 0\n push arg0 d0 d1\n push arg1 d1\n mul\n reduce sum\n store\nend\n"
    r = region(H, text)
    sums = r(x, c, out_shape=(rows,))
    r.close()
    want = torch.cat([(x[r0:r0 + 2048].float() * c.float()).sum(dim=1) for r0 in range(0, rows, 2048)])
    assert torch.equal(sums, want)
    # out[j, i] = x[i, j] + c[j]: the transposed read through LDS tiles
    text = head + "arg out f16 2\nsegment 2\n size arg0.1 arg0.0\n outoff 0\n push arg0 d1 d0\n push arg1 d0\n add\n store\nend\n"
    r = region(H, text)
    out = r(x, c, out_shape=(n, rows))
    r.close()
    for j0 in range(0, n, 8192):
        assert torch.equal(out[j0:j0 + 8192], (x[:, j0:j0 + 8192] + c[j0:j0 + 8192]).t()), j0


@pytest.mark.parametrize("ty,ity", [("f16", "i64"), ("f32", "i32"), ("bf16", "i32")])
def test_column_gather_from_rows_staged_in_lds(H, ty, ity):
    """out[i, j] = relu(data[i, idx[j]]) + bias[j] with rows long enough for the compiled kernel
    that stages each source row in LDS (a workgroup per row); indices out of range give NaN
    and set the flag; a source row of odd length keeps the ordinary kernel.  Bit-exact."""
    import torch
    rng = np.random.default_rng(21)
    text = RC.RELU_COLGATHER_ADD.replace("f16", ty).replace("i64", ity)
    idt = np.int64 if ity == "i64" else np.int32

    def vals(shape):
        v = rng.integers(-4, 5, shape).astype(np.float32)
        return v.astype(np.float16) if ty == "f16" else O.f32_to_bf16_bits(v) if ty == "bf16" else v

    for (m, k, n) in ((5, 4096, 8192), (3, 1000, 4100), (2, 4097, 4096)):
        data, bias = vals((m, k)), vals((n,))
        idx = rng.integers(0, k, (n,)).astype(idt)
        idx[:3] = (0, k - 1, k // 2)
        want = RO.evaluate(text, [data, idx, bias])
        got = run(H, text, [data, idx, bias], (m, n))
        assert got.tobytes() == want.tobytes(), (m, k, n)
    data, bias = vals((4, 2048)), vals((4096,))
    idx = rng.integers(0, 2048, (4096,)).astype(idt)
    idx[7], idx[4000] = 2048, -1
    ws = torch.zeros(2, dtype=torch.int32, device="cuda")
    got = run(H, text, [data, idx, bias], (4, 4096), workspace=ws)
    assert int(ws[0].item()) != 0
    gf = O.bf16_bits_to_f32(got) if ty == "bf16" else got.astype(np.float32)
    assert np.isnan(gf[:, 7]).all() and np.isnan(gf[:, 4000]).all()
    good = np.ones(4096, bool)
    good[[7, 4000]] = False
    idx[[7, 4000]] = 0
    want = RO.evaluate(text, [data, idx, bias])
    assert got[:, good].tobytes() == want[:, good].tobytes()


@pytest.mark.parametrize("ty,ity", [("f16", "i64"), ("f32", "i32")])
def test_column_gather_workgroups_that_walk_several_rows(H, ty, ity):
    """The staged column gather requests a workgroup's (or, for short output rows, a
    wavefront's) next source row while it gathers the current one.  Grids smaller than the number of rows (forced through block_dim, uneven
    shares included, and more rows than the largest grid), a source row that fills the
    look-ahead registers exactly, one chunk more than that (no look-ahead), and a row that
    is not a multiple of 256 chunks.  Bit-exact."""
    rng = np.random.default_rng(33)
    text = RC.RELU_COLGATHER_ADD.replace("f16", ty).replace("i64", ity)
    idt = np.int64 if ity == "i64" else np.int32
    per_chunk = 8 if ty == "f16" else 4

    def vals(shape):
        v = rng.integers(-4, 5, shape).astype(np.float32)
        return v.astype(np.float16) if ty == "f16" else v

    cases = [(10, 1024 * per_chunk, 4096, 3),            # 1024 chunks: all four look-ahead registers of every lane
             (10, 1025 * per_chunk, 4096, 3),            # one chunk more: rows are loaded when their turn comes
             (7, 300 * per_chunk, 8192, 2),              # 300 chunks: some lanes hold two, some one
             (11, 520, 4104, 4),                         # passes that are partly empty
             (4500, 64 * per_chunk, 4096, 0),            # more rows than workgroups in the default grid
             # output rows of at most two passes of a wavefront: the form with a wavefront per row
             # (launched for a thousand rows or more)
             (1033, 64 * per_chunk, 2048, 37), (4500, 32 * per_chunk, 1032, 0), (1030, 256 * per_chunk, 1024, 100),
             (1100, 257 * per_chunk, 2048, 64)]          # ... with a source row beyond its look-ahead registers
    for (m, k, n, block_dim) in cases:
        data, bias = vals((m, k)), vals((n,))
        idx = rng.integers(0, k, (n,)).astype(idt)
        idx[:3] = (0, k - 1, k // 2)
        want = RO.evaluate(text, [data, idx, bias])
        got = run(H, text, [data, idx, bias], (m, n), block_dim=block_dim)
        assert got.tobytes() == want.tobytes(), (m, k, n, block_dim)


def test_unaligned_bases_take_the_element_path(H):
    import torch
    rng = np.random.default_rng(12)
    a = rng.uniform(-2, 2, (17, 40)).astype(np.float16)
    c = rng.uniform(-2, 2, (40,)).astype(np.float16)
    text = RC.HEADER + ("arg in f16 2\narg in f16 1\narg out f16 2\nsegment 2\n size arg0.0 arg0.1\n"
                        " outoff 0\n push arg0 d0 d1\n push arg1 d1\n mul\n store\nend\n")
    want = RO.evaluate(text, [a, c])
    r = region(H, text)
    # same data at odd element offsets: neither operand is 16-byte aligned
    abuf = torch.zeros(a.size + 8, dtype=torch.float16, device="cuda")
    cbuf = torch.zeros(c.size + 8, dtype=torch.float16, device="cuda")
    obuf = torch.zeros(a.size + 8, dtype=torch.float16, device="cuda")
    abuf[3:3 + a.size] = torch.from_numpy(a.ravel()).cuda()
    cbuf[1:1 + c.size] = torch.from_numpy(c).cuda()
    rc = r.launch_raw([abuf.data_ptr() + 6, cbuf.data_ptr() + 2, obuf.data_ptr() + 10],
                      H.pack_tiling(17, 40, 40, 17, 40))
    assert rc == 0
    torch.cuda.synchronize()
    got = obuf[5:5 + a.size].cpu().numpy().reshape(17, 40)
    assert got.tobytes() == want.tobytes()
    assert float(obuf[:5].abs().sum()) == 0 and float(obuf[5 + a.size:].abs().sum()) == 0
    r.close()


def test_special_values_match_the_oracle(H):
    nan, inf = np.float32("nan"), np.float32("inf")
    a = np.array([[-0.0, 0.0, nan, 1.0, -inf, -2.0, inf, 1e-40, -1e-40, 3.0]], dtype=np.float32)
    b = np.array([0.0, -0.0, 1.0, nan, 3.0, -1.0, inf, 2.0, 0.5, 0.0], dtype=np.float32)
    head = RC.HEADER + "arg in f32 2\narg in f32 1\narg out f32 2\nsegment 2\n size arg0.0 arg0.1\n outoff 0\n"
    for body in ("push arg0 d0 d1\n push arg1 d1\n max\n", "push arg0 d0 d1\n push arg1 d1\n min\n",
                 "push arg0 d0 d1\n relu\n", "push arg0 d0 d1\n leaky 0.01\n",
                 "push arg0 d0 d1\n push arg1 d1\n div\n", "push arg0 d0 d1\n push arg1 d1\n mul\n",
                 "push arg0 d0 d1\n push arg1 d1\n sub\n neg\n"):
        text = head + body + " store\nend\n"
        want = RO.evaluate(text, [a, b])
        got = run(H, text, [a, b], a.shape)
        same = (got.view(np.uint32) == want.view(np.uint32)) | (np.isnan(got) & np.isnan(want))
        assert same.all(), (body, got, want)


def test_gather_out_of_range_sets_the_flag_and_reads_nothing_outside(H):
    import torch
    text, inputs, _ = RC.case_relu_colgather_add(8, 64, 24)
    idx = inputs[1].copy()
    idx[5] = 64
    idx[9] = -1
    ws = torch.zeros(4, dtype=torch.int32, device="cuda")
    got = run(H, text, [inputs[0], idx, inputs[2]], (8, 24), workspace=ws)
    assert int(ws[0]) != 0
    assert np.isnan(got[:, 5]).all() and np.isnan(got[:, 9]).all()
    good = [j for j in range(24) if j not in (5, 9)]
    ref = O.relu_colgather_add_f16(inputs[0], np.where((idx < 0) | (idx >= 64), 0, idx), inputs[2])
    assert got[:, good].tobytes() == ref[:, good].tobytes()


OPS2 = ["add", "sub", "mul", "div", "max", "min"]
OPS1 = ["relu", "leaky 0.125", "neg"]


def _random_program(rng, ty):
    """A random chain over x[d0,d1] (identity), r[d0] (row broadcast), c[d1]
    (column broadcast) and t[d1,d0] (transposed)."""
    lines = ["push arg0 d0 d1"]
    depth = 1
    for _ in range(int(rng.integers(2, 9))):
        k = rng.integers(0, 4)
        if depth < 3 and k == 0:
            lines.append(["push arg1 d0", "push arg2 d1", "push arg3 d1 d0", "const 0.75",
                          "dup 0"][int(rng.integers(0, 5))])
            depth += 1
        elif depth >= 2 and k in (1, 2):
            lines.append(OPS2[int(rng.integers(0, len(OPS2)))])
            depth -= 1
        else:
            lines.append(OPS1[int(rng.integers(0, len(OPS1)))])
    while depth > 1:
        lines.append(OPS2[int(rng.integers(0, 3))])
        depth -= 1
    return (RC.HEADER + f"arg in {ty} 2\narg in {ty} 1\narg in {ty} 1\narg in {ty} 2\narg out {ty} 2\n"
            "segment 2\n size arg0.0 arg0.1\n outoff 0\n " + "\n ".join(lines) + "\n store\nend\n")


@pytest.mark.parametrize("seed", range(24))
def test_random_chains_bit_exact(H, seed):
    rng = np.random.default_rng(1000 + seed)
    ty = ["f32", "f16", "bf16"][seed % 3]
    m, n = int(rng.integers(1, 70)), int(rng.integers(1, 200))
    text = _random_program(rng, ty)

    def gen(shape):
        x = rng.uniform(-3, 3, shape).astype(np.float32)
        if ty == "f16":
            return x.astype(np.float16)
        if ty == "bf16":
            return O.f32_to_bf16_bits(x)
        return x
    inputs = [gen((m, n)), gen((m,)), gen((n,)), gen((n, m))]
    want = RO.evaluate(text, inputs)
    got = run(H, text, inputs, (m, n))
    if ty == "bf16":
        wf, gf = O.bf16_bits_to_f32(want), O.bf16_bits_to_f32(got)
    else:
        wf, gf = want.astype(np.float32), got.astype(np.float32)
    same = (got.view(np.uint16 if ty != "f32" else np.uint32) ==
            want.view(np.uint16 if ty != "f32" else np.uint32)) | (np.isnan(wf) & np.isnan(gf))
    assert same.all(), text


@pytest.mark.parametrize("name", sorted(RC.INT_CASES))
def test_integer_regions_bit_exact(H, name):
    """i16 / i32 regions on full-range values (wraparound, 16-bit comparisons,
    mixed widths, gathered rows, a transposed read): equal to numpy's fixed-width
    arithmetic and to the region oracle."""
    text, inputs, want = RC.INT_CASES[name]()
    assert RO.evaluate(text, inputs).tobytes() == want.tobytes()
    got = run(H, text, inputs, want.shape)
    assert got.dtype == want.dtype and got.tobytes() == want.tobytes()


INT_OPS2 = ["add", "sub", "mul", "max", "min"]
INT_OPS1 = ["relu", "neg"]


@pytest.mark.parametrize("seed", range(12))
def test_random_integer_chains_bit_exact(H, seed):
    """Seeded random integer programs over an identity read, a row and a column
    broadcast and a transposed read, on ragged shapes."""
    rng = np.random.default_rng(5000 + seed)
    ty = ["i32", "i16"][seed % 2]
    dt = np.int32 if ty == "i32" else np.int16
    lines, depth = ["push arg0 d0 d1"], 1
    for _ in range(int(rng.integers(2, 9))):
        k = rng.integers(0, 4)
        if depth < 3 and k == 0:
            lines.append(["push arg1 d0", "push arg2 d1", "push arg3 d1 d0", "const -3", "dup 0"][int(rng.integers(0, 5))])
            depth += 1
        elif depth >= 2 and k in (1, 2):
            lines.append(INT_OPS2[int(rng.integers(0, len(INT_OPS2)))])
            depth -= 1
        else:
            lines.append(INT_OPS1[int(rng.integers(0, len(INT_OPS1)))])
    while depth > 1:
        lines.append(INT_OPS2[int(rng.integers(0, 3))])
        depth -= 1
    text = (RC.HEADER + f"arg in {ty} 2\narg in {ty} 1\narg in {ty} 1\narg in {ty} 2\narg out {ty} 2\n"
            "segment 2\n size arg0.0 arg0.1\n outoff 0\n " + "\n ".join(lines) + "\n store\nend\n")
    m, n = int(rng.integers(1, 70)), int(rng.integers(1, 200))
    # small magnitudes half of the time so that comparisons are not all decided by overflow
    lim = np.iinfo(dt).max if seed % 4 < 2 else 50
    inputs = [rng.integers(-lim, lim, shape, dtype=dt, endpoint=True) for shape in ((m, n), (m,), (n,), (n, m))]
    want = RO.evaluate(text, inputs)
    got = run(H, text, inputs, (m, n))
    assert got.dtype == want.dtype and got.tobytes() == want.tobytes(), text


def test_integer_unaligned_views_and_tails(H):
    """Integer tensors at odd element offsets (no 128-bit access possible) and rows
    with tails, against the oracle."""
    import torch
    rng = np.random.default_rng(9)
    for ty, dt in (("i32", np.int32), ("i16", np.int16)):
        text = RC.INT_ADD_I32.replace("i32", ty)
        for m, n in ((1, 1), (3, 19), (5, 64), (2, 4099)):
            a = rng.integers(np.iinfo(dt).min, np.iinfo(dt).max, (m, n), dtype=dt)
            b = rng.integers(np.iinfo(dt).min, np.iinfo(dt).max, (m, n), dtype=dt)
            want = RO.evaluate(text, [a, b])
            r = region(H, text)
            da = torch.zeros(m * n + 1, dtype=getattr(torch, "int32" if ty == "i32" else "int16"), device="cuda")
            da[1:] = torch.from_numpy(a.reshape(-1)).cuda()
            got = r(da[1:].view(m, n), _dev(b, ty), out_shape=(m, n)).cpu().numpy()
            r.close()
            assert got.tobytes() == want.tobytes(), (ty, m, n)


def _random_region(rng, extras=False):
    """A random program with its inputs and output shape: iteration rank 1..3; operands
    read whole, broadcast along rows or columns, transposed or gathered; one element type
    or a mix; elementwise or a row sum; extents drawn from the classes the kernels tell
    apart (short rows, whole vectors with partly empty passes, whole passes, ragged).
    extras: also roundings to a narrower type in the chain and, in elementwise programs,
    extent constants (the runtime extent of an argument as a value)."""
    rank = int(rng.integers(1, 4))
    reduce = rank >= 2 and rng.random() < 0.35
    types = [["f32"], ["f16"], ["bf16"], ["f16", "f32"]][int(rng.integers(0, 4))]
    n = int(rng.choice([1, 5, 8, 24, 40, 64, 96, 250, 256, 1000, 1024, 2048, 4096, 4099]))
    if rank == 1:
        n = int(rng.choice([7, 64, 1000, 33000, 70001]))
    outer = [int(rng.choice([1, 2, 3, 17, 64, 130]))] if rank >= 2 else []
    if rank == 3:
        outer.append(int(rng.choice([1, 4, 9])))
    size = outer + [n]
    last = rank - 1
    dims = lambda ks: " ".join(f"d{k}" for k in ks)
    # (map text, tensor shape) of the operand kinds available at this rank
    kinds = [(dims(range(rank)), tuple(size)), (f"d{last}", (n,))]
    if rank >= 2:
        kinds.append((dims(range(rank - 1)), tuple(size[:-1])))               # the same along a row
        kinds.append((f"d{last - 1} d{last}" if rank == 3 else f"d0 0", (size[last - 1], n) if rank == 3 else (size[0], 1)))
    if rank == 2 and not reduce:
        kinds.append(("d1 d0", (n, size[0])))                                  # transposed
    if rank == 3 and not reduce:
        kinds.append(("d0 d2 d1", (size[0], n, size[1])))
    args, shapes, pushes = [f"arg in {types[0]} {rank}"], [tuple(size)], []
    ops = ["push arg0 " + dims(range(rank))]
    gather = rank == 2 and rng.random() < 0.25
    if gather:                                   # rows of a table picked by an index tensor
        table_rows = int(rng.integers(size[0], size[0] + 50))
        ity = ["i32", "i64"][int(rng.integers(0, 2))]
        args += [f"arg in {types[-1]} 2", f"arg in {ity} 1"]
        shapes += [(table_rows, n), ("index", ity, table_rows, size[0])]
        ops += [f"push arg1 g0:arg2 d1", "add"]
    depth = 1
    allowed2 = ["add", "sub", "mul", "max", "min"] + ([] if reduce else ["div"])
    allowed1 = ["relu", "neg"] + ([] if reduce else ["leaky 0.25"])
    if extras:
        allowed1 += ["cast f16", "cast bf16"]
    for _ in range(int(rng.integers(1, 7))):
        k = int(rng.integers(0, 4))
        if depth < 3 and k == 0 and len(args) < 6:
            if extras and not reduce and rng.random() < 0.3:
                ops.append(f"const arg0.{int(rng.integers(0, rank))} {['f32', 'f16', 'bf16'][int(rng.integers(0, 3))]}")
            elif rng.random() < 0.2:
                ops.append("const 2")
            else:
                text, shape = kinds[int(rng.integers(0, len(kinds)))]
                ty = types[int(rng.integers(0, len(types)))]
                ops.append(f"push arg{len(args)} {text}")
                args.append(f"arg in {ty} {len(shape)}")
                shapes.append(shape)
            depth += 1
        elif depth >= 2 and k in (1, 2):
            ops.append(allowed2[int(rng.integers(0, len(allowed2)))])
            depth -= 1
        else:
            ops.append(allowed1[int(rng.integers(0, len(allowed1)))])
    while depth > 1:
        ops.append(["add", "sub", "max"][int(rng.integers(0, 3))])
        depth -= 1
    out_ty = types[0]
    out_shape = tuple(size[:-1]) if reduce else tuple(size)
    text = (RC.HEADER + "\n".join(args) + f"\narg out {out_ty} {len(out_shape)}\nsegment {rank}\n size "
            + " ".join(f"arg0.{k}" for k in range(rank)) + "\n outoff 0\n " + "\n ".join(ops)
            + ("\n reduce sum" if reduce else "") + "\n store\nend\n")
    inputs = []
    for a, shape in zip(args, shapes):
        ty = a.split()[2]
        if shape and shape[0] == "index":
            _, ity, hi, count = shape
            inputs.append(rng.integers(0, hi, (count,)).astype(np.int32 if ity == "i32" else np.int64))
            continue
        v = rng.integers(-3, 4, shape).astype(np.float32)           # small integers: sums are exact in any order
        inputs.append(v.astype(np.float16) if ty == "f16" else O.f32_to_bf16_bits(v) if ty == "bf16" else v)
    return text, inputs, out_shape, out_ty


@pytest.mark.parametrize("seed", range(60 + 40))
def test_random_programs_over_the_shape_classes(H, seed):
    """(seeds from 60 on: with roundings in the chain and extent constants)"""
    rng = np.random.default_rng(777 + seed)
    text, inputs, out_shape, out_ty = _random_region(rng, extras=seed >= 60)
    want = RO.evaluate(text, inputs)
    got = run(H, text, inputs, out_shape)
    if out_ty == "bf16":
        wf, gf = O.bf16_bits_to_f32(want), O.bf16_bits_to_f32(got)
    else:
        wf, gf = want.astype(np.float32), got.astype(np.float32)
    bits = np.uint32 if out_ty == "f32" else np.uint16
    same = (got.view(bits) == want.view(bits)) | (np.isnan(wf) & np.isnan(gf))
    assert same.all(), (text, [getattr(x, "shape", None) for x in inputs], np.argwhere(~same)[:5])


def test_every_operation_pair_at_every_vector_position(H):
    """binary step followed by up to two activations, all combinations, on rows
    of 19 elements (two full vectors and a tail): every position of the result
    must match the oracle."""
    rng = np.random.default_rng(77)
    a = rng.uniform(-3, 3, (3, 19)).astype(np.float32)
    b = rng.uniform(-3, 3, (19,)).astype(np.float32)
    head = RC.HEADER + "arg in f32 2\narg in f32 1\narg out f32 2\nsegment 2\n size arg0.0 arg0.1\n outoff 0\n"
    unaries = ["", "relu\n", "leaky 0.25\n", "neg\n"]
    for first in (" push arg0 d0 d1\n push arg1 d1\n", " push arg1 d1\n push arg0 d0 d1\n"):
        for op in OPS2:
            for u1 in unaries:
                for u2 in unaries:
                    text = head + first + f" {op}\n {u1} {u2} store\nend\n"
                    want = RO.evaluate(text, [a, b])
                    got = run(H, text, [a, b], a.shape)
                    same = (got.view(np.uint32) == want.view(np.uint32)) | (np.isnan(got) & np.isnan(want))
                    assert same.all(), (text, np.argwhere(~same))


def test_code_object_of_another_program_is_rejected(H, evaluator, tmp_path):
    """A code object carries the hash of the program it was emitted from; the
    first launch checks it and runs nothing when it does not match."""
    import torch
    if evaluator != "compiled":
        pytest.skip("one run is enough")
    other = H.Region(RC.RELU_COL_ADD)
    image = H.compile_region_source(other.emit_source(), str(tmp_path))
    other.close()
    r = H.Region(RC.C1_ADD_MUL)
    r.attach_code_object(image)
    a = torch.ones(4, 8, device="cuda")
    with pytest.raises(H.AfirHipError, match="not built from this program"):
        r(a, a, out_shape=(4, 8))
    r.close()


def test_code_object_of_another_emitter_version_is_rejected(H, evaluator, monkeypatch, tmp_path):
    """The code object also carries the version of the kernel set and launch arguments it
    was emitted for; one from another version (here: the source edited) is refused when it
    is loaded, before any of its kernels is launched."""
    import re
    import torch
    if evaluator != "compiled":
        pytest.skip("one run is enough")
    monkeypatch.setenv("AFIR_HIP_REGION_GENERIC", "1")
    r = H.Region(RC.C1_ADD_MUL)
    src = r.emit_source()
    assert re.search(r"afir_region_emit_abi = \d+;", src)
    for edited in (re.sub(r"afir_region_emit_abi = \d+;", "afir_region_emit_abi = 1;", src),
                   re.sub(r"afir_region_emit_abi = ", "afir_region_other = ", src)):      # another version, none
        r.attach_code_object(H.compile_region_source(edited, str(tmp_path)))
        a = torch.ones(4, 8, device="cuda")
        with pytest.raises(H.AfirHipError, match="another version of this library"):
            r(a, a, out_shape=(4, 8))
    r.close()


def test_preferred_code_object_outranks_a_hand_tuned_family(H, evaluator, monkeypatch, tmp_path):
    """A program that is exactly one of the hand-tuned families keeps that kernel
    when a code object is attached, unless the code object is preferred."""
    import torch
    if evaluator != "compiled":
        pytest.skip("one run is enough")
    monkeypatch.setenv("AFIR_HIP_REGION_GENERIC", "0")
    text, inputs, want = RC.case_c3()
    r = H.Region(text)
    assert r.kernel == "relu_broadcast_add_transpose"
    r.compile(cache_dir=str(tmp_path))
    assert r.kernel == "relu_broadcast_add_transpose"
    r.prefer_code_object()
    assert r.kernel == "fused_region_compiled"
    got = r(*[torch.from_numpy(x).cuda() for x in inputs], out_shape=want.shape).cpu().numpy()
    assert got.tobytes() == want.tobytes()
    r.prefer_code_object(False)
    assert r.kernel == "relu_broadcast_add_transpose"
    r.close()


def test_split_row_sums_launched_from_two_streams_do_not_mix_their_partial_sums(H, evaluator):
    """A handful of very long rows is summed by a split kernel and a join kernel that share
    the code object's partial sums.  Launches of that form from different streams are chained
    by the library (the second waits for the first one's join): alternating two streams and
    two inputs, every result must be its own input's."""
    import torch
    if evaluator != "compiled":
        pytest.skip("the split / join form belongs to the compiled kernels")
    text = RC.C2_BCAST_ADD_ROWSUM
    rows, n = 16, 1 << 20
    rng = np.random.default_rng(5)
    xs = [torch.from_numpy(rng.integers(-4, 5, (rows, n)).astype(np.float32)).cuda() for _ in range(2)]
    bias = torch.from_numpy(rng.integers(-4, 5, (n,)).astype(np.float32)).cuda()
    want = [(x.double().sum(1) + bias.double().sum()).cpu().numpy().astype(np.float32) for x in xs]
    r = region(H, text)
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    outs = [[torch.empty((rows,), dtype=torch.float32, device="cuda") for _ in range(6)] for _ in range(2)]
    tiling = H.pack_tiling(rows, n, n, rows)
    torch.cuda.synchronize()
    for k in range(6):
        for i in range(2):
            rc = r.launch_raw([xs[i].data_ptr(), bias.data_ptr(), outs[i][k].data_ptr()], tiling,
                              stream=streams[i].cuda_stream)
            assert rc == 0
    torch.cuda.synchronize()
    for i in range(2):
        for k in range(6):
            assert np.array_equal(outs[i][k].cpu().numpy(), want[i]), (i, k)
    r.close()
