"""Compiled region kernels that separate the chip's reads from its writes in time
(afir_region_s<k>_phased_i32, afir_region_all_phased_i32): taken for parallel segments of one
or two streamed operands at shapes of whole workgroups between 16 and 128 MiB of output.
Every case is compared bit for bit with the region oracle and with the same code object kept
off those kernels (AFIR_HIP_REGION_PHASED=0), and the kernel that ran is checked by name.
Reference semantics of the regions: lib/Conversion/LinalgToAscendC/ComputeConversion.cpp:
1290-1640 (parallel generics, inlined bodies), :828-1272 (the fused gather).  Needs a GPU and hipcc."""
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


@pytest.fixture(scope="module")
def cache(tmp_path_factory):
    return str(tmp_path_factory.mktemp("phased_cache"))


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


def run_both(H, cache, monkeypatch, text, inputs, out_shape, kernel, workgroups=None, workspace=None):
    """(phased result, unphased result) as host arrays; checks which kernel each launch took."""
    monkeypatch.setenv("AFIR_HIP_REGION_GENERIC", "1")
    r = H.Region(text).compile(cache_dir=cache)
    dev = [_dev(x, r.arg_types[i]) for i, x in enumerate(inputs)]
    monkeypatch.delenv("AFIR_HIP_REGION_PHASED", raising=False)
    got = _host(r(*dev, out_shape=out_shape, workspace=workspace), r.arg_types[-1])
    note = H.last_launch()
    assert note["kernel"] == kernel, note
    if workgroups is not None:
        assert note["workgroups"] == workgroups, note
    monkeypatch.setenv("AFIR_HIP_REGION_PHASED", "0")
    plain = _host(r(*dev, out_shape=out_shape, workspace=workspace), r.arg_types[-1])
    assert "phased" not in H.last_launch()["kernel"]
    monkeypatch.delenv("AFIR_HIP_REGION_PHASED")
    r.close()
    return got, plain


def test_two_streamed_inputs_in_two_rounds(H, cache, monkeypatch):
    """(a + b) * b, f32 [2048, 4096]: 32 MiB of output, rows of 1024 groups (128 lanes per row)."""
    rng = np.random.default_rng(1)
    a = rng.uniform(-1, 1, (2048, 4096)).astype(np.float32)
    b = rng.uniform(-1, 1, (2048, 4096)).astype(np.float32)
    got, plain = run_both(H, cache, monkeypatch, RC.C1_ADD_MUL, [a, b], a.shape, "afir_region_s0_phased_i32", 1024)
    want = (a + b) * b
    assert got.tobytes() == want.tobytes() and plain.tobytes() == want.tobytes()


@pytest.mark.parametrize("nidx", [16384, 32768 + 8192])       # one launch; two launches of 1280 workgroups
def test_gathered_rows_with_row_vectors_in_lds(H, cache, monkeypatch, nidx):
    """table[idx] * scale + shift, f16 rows of 1024: the gathered rows are the streamed operand,
    scale and shift are staged in LDS once per workgroup.  A bad index gives a NaN row and sets
    the workspace flag, as on the other kernels."""
    import torch
    rng = np.random.default_rng(2)
    table = (rng.standard_normal((5000, 1024)) * 0.02).astype(np.float16)
    idx = rng.integers(0, 5000, nidx).astype(np.int32)
    scale = rng.uniform(0.5, 1.5, 1024).astype(np.float16)
    shift = rng.uniform(-0.1, 0.1, 1024).astype(np.float16)
    want = RO.evaluate(RC.C4_GATHER_SCALE_SHIFT, [table, idx, scale, shift])
    grid = 1024 if nidx == 16384 else 1280
    got, plain = run_both(H, cache, monkeypatch, RC.C4_GATHER_SCALE_SHIFT, [table, idx, scale, shift], (nidx, 1024),
                          "afir_region_s0_phased_i32", grid)
    assert got.tobytes() == want.tobytes() and plain.tobytes() == want.tobytes()
    idx[[5, nidx - 1]] = [5000, -3]
    ws = torch.zeros(4, dtype=torch.int32, device="cuda")
    got, plain = run_both(H, cache, monkeypatch, RC.C4_GATHER_SCALE_SHIFT, [table, idx, scale, shift], (nidx, 1024),
                          "afir_region_s0_phased_i32", grid, workspace=ws)
    assert int(ws[0].item()) != 0
    assert np.isnan(got[[5, nidx - 1]]).all() and got.tobytes() == plain.tobytes()


def test_every_segment_of_a_program_in_one_phased_launch(H, cache, monkeypatch):
    """The reference's split / relu / broadcast graph at [8192, 4096] f16: two segments of 32 MiB,
    each with a value per row and a row vector, together one launch of 2048 workgroups."""
    rng = np.random.default_rng(3)
    x = rng.uniform(-1, 1, (8192, 4096)).astype(np.float16)
    b0, b1 = (rng.uniform(-1, 1, 4096).astype(np.float16) for _ in range(2))
    s0, s1 = (rng.uniform(-1, 1, 4096).astype(np.float16) for _ in range(2))
    inputs = [x, b0, b1, s0, s1]
    want = RO.evaluate(RC.SPLIT_RELU_BRC_ADD_MUL, inputs)
    got, plain = run_both(H, cache, monkeypatch, RC.SPLIT_RELU_BRC_ADD_MUL, inputs, x.shape, "afir_region_all_phased_i32", 2048)
    assert got.tobytes() == want.tobytes() and plain.tobytes() == want.tobytes()


COPY_RANK1 = RC.HEADER + "arg in bf16 1\narg out bf16 1\nsegment 1\n size arg0.0\n outoff 0\n push arg0 d0\n const 0.5\n mul\n store\nend\n"
INT_CHAIN = RC.HEADER + ("arg in i32 2\narg in i32 1\narg out i32 2\nsegment 2\n size arg0.0 arg0.1\n outoff 0\n"
                         " push arg0 d0 d1\n push arg1 d0\n add\n relu\n store\nend\n")


def test_long_rows_integers_and_the_hold_from_the_environment(H, cache, monkeypatch):
    """A rank-1 tensor (one row of 2^22 groups: 2048 stretches, a workgroup each), an integer
    region with a value per row, and holds far too short and far too long: timing only."""
    rng = np.random.default_rng(4)
    x = rng.integers(0, 1 << 16, 1 << 25).astype(np.uint16)          # bf16 bit patterns, NaN and inf among them
    want = RO.evaluate(COPY_RANK1, [x])
    got, plain = run_both(H, cache, monkeypatch, COPY_RANK1, [x], x.shape, "afir_region_s0_phased_i32", 2048)
    assert got.tobytes() == want.tobytes() and plain.tobytes() == want.tobytes()
    a = rng.integers(-2 ** 31, 2 ** 31, (4096, 2048)).astype(np.int32)
    b = rng.integers(-2 ** 31, 2 ** 31, 4096).astype(np.int32)
    want = RO.evaluate(INT_CHAIN, [a, b])
    for gbs, base in ((None, None), ("100000", "0"), ("500", "20000")):
        if gbs:
            monkeypatch.setenv("AFIR_REGION_PHASE_GBS", gbs)
            monkeypatch.setenv("AFIR_REGION_PHASE_BASE_NS", base)
        got, plain = run_both(H, cache, monkeypatch, INT_CHAIN, [a, b], a.shape, "afir_region_s0_phased_i32", 1024)
        assert got.tobytes() == want.tobytes() and plain.tobytes() == want.tobytes()


def test_shapes_outside_the_phased_form_keep_to_the_other_kernels(H, cache, monkeypatch):
    """Too small, rows that are not whole workgroups, a caller-given grid: not phased, same bits."""
    monkeypatch.setenv("AFIR_HIP_REGION_GENERIC", "1")
    rng = np.random.default_rng(5)
    r = H.Region(RC.C1_ADD_MUL).compile(cache_dir=cache)
    for shape, block_dim in (((256, 4096), 0), ((2049, 4096), 0), ((2048, 4100), 0), ((2048, 4096), 64)):
        a = rng.uniform(-1, 1, shape).astype(np.float32)
        b = rng.uniform(-1, 1, shape).astype(np.float32)
        out = r(_dev(a, "f32"), _dev(b, "f32"), out_shape=shape, block_dim=block_dim).cpu().numpy()
        assert "phased" not in H.last_launch()["kernel"], shape
        assert out.tobytes() == ((a + b) * b).tobytes(), shape
    r.close()


@pytest.mark.parametrize("name", ["c1", "c3", "c4", "relu_colgather_add", "split_relu_brc_add_mul", "cast_chain_f16",
                                  "reduce_rowbias", "mean_rowbias"])
def test_regions_compiled_inside_the_process_give_the_same_bits(H, cache, monkeypatch, name):
    """afir_hip_region_compile (the HIP runtime's compiler library, no hipcc) against the code
    object hipcc builds from the same source: the same output, bit for bit, and (for the
    elementwise cases) the oracle's."""
    monkeypatch.setenv("AFIR_HIP_REGION_GENERIC", "1")
    exact = name in RC.EXACT_CASES
    text, inputs, want = (RC.EXACT_CASES if exact else RC.REDUCE_CASES)[name]()
    outs = []
    for in_process in (True, False):
        r = H.Region(text).compile(cache_dir=cache, in_process=in_process)
        assert r.kernel == "fused_region_compiled"
        dev = [_dev(x, r.arg_types[i]) for i, x in enumerate(inputs)]
        outs.append(_host(r(*dev, out_shape=want.shape), r.arg_types[-1]))
        r.close()
    assert outs[0].tobytes() == outs[1].tobytes()
    if exact:
        assert outs[0].tobytes() == want.tobytes()


def _random_phased_program(rng):
    """A random elementwise program of the form the phased kernels take: one or two operands
    streamed with the output, row vectors, per-row values and constants, all of one element size,
    roundings and extent constants among the operations; rank 2 or 3, 16-64 MiB of output."""
    ty = ["f32", "f16", "bf16"][int(rng.integers(0, 3))]
    esize = 4 if ty == "f32" else 2
    rank = int(rng.integers(2, 4))
    n = int(rng.choice([1024, 2048, 4096, 8192]))                 # row length: 8 * 2^k groups
    rows = (int(rng.choice([16, 32, 48])) << 20) // (n * esize)   # 16 / 32 / 48 MiB of output
    size = [rows, n] if rank == 2 else [4, rows // 4, n]
    last = rank - 1
    dims = " ".join(f"d{k}" for k in range(rank))
    kinds = [(dims, tuple(size)), (f"d{last}", (n,)), (" ".join(f"d{k}" for k in range(last)), tuple(size[:-1]))]
    args, shapes = [f"arg in {ty} {rank}"], [tuple(size)]
    ops = [f"push arg0 {dims}"]
    depth, streamed, vectors = 1, 1, 0
    for _ in range(int(rng.integers(2, 8))):
        k = int(rng.integers(0, 4))
        if depth < 3 and k == 0 and len(args) < 5:
            pick = int(rng.integers(0, 5))
            if pick == 0:
                ops.append("const 1.5")
            elif pick == 1:
                ops.append(f"const arg0.{int(rng.integers(0, rank))} f32")
            else:
                which = int(rng.choice([0, 1, 1, 2])) if streamed < 2 else int(rng.choice([1, 1, 2]))
                text, shape = kinds[which]
                streamed += which == 0
                vectors += which == 1
                ops.append(f"push arg{len(args)} {text}")
                args.append(f"arg in {ty} {len(shape)}")
                shapes.append(shape)
            depth += 1
        elif depth >= 2 and k in (1, 2):
            ops.append(["add", "sub", "mul", "max", "min", "div"][int(rng.integers(0, 6))])
            depth -= 1
        else:
            ops.append(["relu", "neg", "leaky 0.25", "cast f16", "cast bf16"][int(rng.integers(0, 5))])
    while depth > 1:
        ops.append(["add", "sub", "max"][int(rng.integers(0, 3))])
        depth -= 1
    text = (RC.HEADER + "\n".join(args) + f"\narg out {ty} {rank}\nsegment {rank}\n size "
            + " ".join(f"arg0.{k}" for k in range(rank)) + "\n outoff 0\n " + "\n ".join(ops) + "\n store\nend\n")
    inputs = []
    for shape in shapes:
        v = rng.uniform(-2, 2, shape).astype(np.float32)
        inputs.append(v if ty == "f32" else v.astype(np.float16) if ty == "f16" else O.f32_to_bf16_bits(v))
    # row vectors are staged in LDS, 16 KiB of them at most
    return text, inputs, tuple(size), ty, vectors * n * esize <= 16384


@pytest.mark.parametrize("seed", range(16))
def test_random_programs_at_phased_shapes(H, cache, monkeypatch, seed):
    """Random chains at shapes the phased kernels take, bit for bit against the oracle, with the
    phased kernels on (checked by name) and off."""
    monkeypatch.setenv("AFIR_HIP_REGION_GENERIC", "1")
    rng = np.random.default_rng(4000 + seed)
    text, inputs, out_shape, ty, fits = _random_phased_program(rng)
    with np.errstate(all="ignore"):
        want = RO.evaluate(text, inputs)
    r = H.Region(text).compile(cache_dir=cache)
    dev = [_dev(x, r.arg_types[i]) for i, x in enumerate(inputs)]
    results = []
    for phased in (None, "0"):
        if phased is None:
            monkeypatch.delenv("AFIR_HIP_REGION_PHASED", raising=False)
        else:
            monkeypatch.setenv("AFIR_HIP_REGION_PHASED", phased)
        results.append(_host(r(*dev, out_shape=out_shape), r.arg_types[-1]))
        if phased is None:
            assert (H.last_launch()["kernel"] == "afir_region_s0_phased_i32") == fits, (text, H.last_launch())
    r.close()
    bits = np.uint32 if ty == "f32" else np.uint16
    wf = O.bf16_bits_to_f32(want) if ty == "bf16" else want.astype(np.float32)
    for got in results:
        gf = O.bf16_bits_to_f32(got) if ty == "bf16" else got.astype(np.float32)
        same = (got.view(bits) == want.view(bits)) | (np.isnan(wf) & np.isnan(gf))
        assert same.all(), (text, np.argwhere(~same)[:5])


def test_a_code_object_can_be_loaded_ahead_of_the_first_launch(H, cache):
    """afir_hip_region_load: nothing attached is nothing to do; an attached code object is loaded
    and checked against the program now (what the first launch would otherwise do), so an image
    built from another program is refused here, before anything is launched."""
    import ctypes
    L = H.load()
    L.afir_hip_region_load.restype = ctypes.c_uint32
    L.afir_hip_region_load.argtypes = [ctypes.c_uint64]
    r = H.Region(RC.C1_ADD_MUL)
    assert L.afir_hip_region_load(ctypes.c_uint64(r.handle)) == 0          # the interpreter needs no loading
    r.compile(cache_dir=cache)
    assert L.afir_hip_region_load(ctypes.c_uint64(r.handle)) == 0
    assert L.afir_hip_region_load(ctypes.c_uint64(r.handle)) == 0          # already loaded
    other = H.Region(RC.RELU_COL_ADD)
    image = H.compile_region_source(r.emit_source(), cache)
    other.attach_code_object(image)
    assert L.afir_hip_region_load(ctypes.c_uint64(other.handle)) != 0
    assert b"not built from this program" in L.afir_hip_last_error()
    assert L.afir_hip_region_load(ctypes.c_uint64(987654321)) != 0
    r.close()
    other.close()
