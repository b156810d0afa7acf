"""The region-program oracle against the closed-form goldens of the reference's
examples and of the benchmark configurations, and the host side of the region
C ABI (parse / validate / resolve) -- CPU only."""
import ctypes
import struct

import numpy as np
import pytest

from oracle import region_oracle as RO
from tests import region_cases as RC


@pytest.mark.parametrize("name", sorted(RC.EXACT_CASES))
def test_program_reproduces_closed_form_golden(name):
    text, inputs, want = RC.EXACT_CASES[name]()
    got = RO.evaluate(text, inputs)
    assert got.dtype == want.dtype and got.shape == want.shape
    assert got.tobytes() == want.tobytes()


@pytest.mark.parametrize("name", sorted(RC.REDUCE_CASES))
def test_reduce_program_reproduces_golden(name):
    text, inputs, want = RC.REDUCE_CASES[name]()
    got = RO.evaluate(text, inputs)
    # same numpy pairwise float32 sum as the golden: identical
    assert got.tobytes() == want.tobytes()


def _py(op, a, b):
    """One float32 operation through Python doubles, rounded with struct
    (a double holds the exact sum / product / difference of two floats, and
    the correctly rounded quotient rounds to the same float)."""
    r = {"add": a + b, "sub": a - b, "mul": a * b, "div": a / b}[op]
    return struct.unpack("<f", struct.pack("<f", r))[0]


@pytest.mark.parametrize("op", ["add", "sub", "mul", "div"])
def test_single_ops_against_python_floats(op):
    rng = np.random.default_rng(3)
    a = rng.uniform(-4, 4, (5, 7)).astype(np.float32)
    b = rng.uniform(0.5, 4, (7,)).astype(np.float32)
    text = RC.HEADER + f"""
arg in f32 2
arg in f32 1
arg out f32 2
segment 2
  size arg0.0 arg0.1
  outoff 0
  push arg0 d0 d1
  push arg1 d1
  {op}
  store
end
"""
    got = RO.evaluate(text, [a, b])
    for i in range(5):
        for j in range(7):
            assert got[i, j] == np.float32(_py(op, float(a[i, j]), float(b[j])))


def test_max_min_relu_special_values():
    nan, inf = np.float32("nan"), np.float32("inf")
    a = np.array([[-0.0, 0.0, nan, 1.0, -inf, -2.0]], dtype=np.float32)
    b = np.array([0.0, -0.0, 1.0, nan, 3.0, -1.0], dtype=np.float32)
    body = "push arg0 d0 d1\n  push arg1 d1\n  {}\n  store"
    head = RC.HEADER + "arg in f32 2\narg in f32 1\narg out f32 2\nsegment 2\n  size arg0.0 arg0.1\n  outoff 0\n  "
    mx = RO.evaluate(head + body.format("max") + "\nend\n", [a, b])[0]
    mn = RO.evaluate(head + body.format("min") + "\nend\n", [a, b])[0]
    assert not np.signbit(mx[0]) and not np.signbit(mx[1])       # max(-0, +0) = +0 either way
    assert np.signbit(mn[0]) and np.signbit(mn[1])               # min(-0, +0) = -0 either way
    assert np.isnan(mx[2]) and np.isnan(mx[3]) and np.isnan(mn[2]) and np.isnan(mn[3])
    assert mx[4] == 3.0 and mn[4] == -inf and mx[5] == -1.0 and mn[5] == -2.0
    relu = RO.evaluate(head + "push arg0 d0 d1\n  relu\n  store\nend\n", [a, b])[0]
    assert not np.signbit(relu[0]) and relu[0] == 0 and np.isnan(relu[2]) and relu[4] == 0 and relu[5] == 0


def test_gather_out_of_range_is_an_error():
    text, inputs, _ = RC.case_relu_colgather_add(4, 10, 6)
    inputs[1] = inputs[1].copy()
    inputs[1][2] = 10
    with pytest.raises(RO.RegionError):
        RO.evaluate(text, inputs)


@pytest.mark.parametrize("name", sorted(RC.INT_CASES))
def test_integer_programs_reproduce_fixed_width_numpy(name):
    """Integer regions against numpy's own int16 / int32 array arithmetic (which
    wraps at the element width), on full-range values with the extremes seeded in."""
    text, inputs, want = RC.INT_CASES[name]()
    got = RO.evaluate(text, inputs)
    assert got.dtype == want.dtype and got.tobytes() == want.tobytes()


def test_integer_wraparound_by_hand():
    """The corners a dropped wrap or a wrong width would miss, written out."""
    head = RC.HEADER + "arg in {t} 1\narg in {t} 1\narg out {t} 1\nsegment 1\n size arg0.0\n outoff 0\n push arg0 d0\n push arg1 d0\n"
    tail = " store\nend\n"
    a32 = np.array([2147483647, -2147483648, 65536, -5], dtype=np.int32)
    b32 = np.array([1, -1, 65536, 3], dtype=np.int32)
    assert RO.evaluate(head.format(t="i32") + " add\n" + tail, [a32, b32]).tolist() == [-2147483648, 2147483647, 131072, -2]
    assert RO.evaluate(head.format(t="i32") + " mul\n" + tail, [a32, b32]).tolist() == [2147483647, -2147483648, 0, -15]
    assert RO.evaluate(head.format(t="i32") + " sub\n neg\n" + tail, [a32, b32]).tolist() == [-2147483646, 2147483647, 0, 8]
    a16 = np.array([32767, -32768, 256, -5], dtype=np.int16)
    b16 = np.array([1, -1, 256, 3], dtype=np.int16)
    assert RO.evaluate(head.format(t="i16") + " add\n" + tail, [a16, b16]).tolist() == [-32768, 32767, 512, -2]
    # the sum wraps to -32768 before the comparison sees it
    assert RO.evaluate(head.format(t="i16") + " add\n relu\n" + tail, [a16, b16]).tolist() == [0, 32767, 512, 0]
    assert RO.evaluate(head.format(t="i16") + " mul\n const 7\n max\n" + tail, [a16, b16]).tolist() == [32767, 7, 7, 7]
    assert RO.evaluate(head.format(t="i16") + " neg\n" + tail.replace(" store", " add\n store"), [a16, b16]).tolist() == \
        [32766, -32767, 0, -8]


# ---- the C ABI's host side: parse / validate / resolve, no GPU needed --------

@pytest.fixture(scope="module")
def H(pkg):
    from ascend_mlir_amd import hip_kernels
    hip_kernels.load()
    return hip_kernels


ALL_TEXTS = {k: getattr(RC, k) for k in dir(RC) if k.isupper() and k != "HEADER"
             and isinstance(getattr(RC, k), str)}


@pytest.mark.parametrize("name", sorted(ALL_TEXTS))
def test_library_accepts_every_case_program(H, name):
    r = H.Region(ALL_TEXTS[name])
    prog = RO.parse(ALL_TEXTS[name])
    assert r.num_inputs == len(prog["args"]) - 1 and r.num_outputs == 1
    want = [f"dim_arg{a}_{d}" for a, (_, _, rank) in enumerate(prog["args"]) for d in range(rank)]
    assert r.tiling_fields == want
    r.close()


def test_library_resolves_shapes_and_rejects_inconsistent_ones(H):
    r = H.Region(RC.SPLIT_RELU_BRC_ADD_MUL)
    ok = H.pack_tiling(640, 512, 320, 320, 512, 512, 640, 512)
    assert r.argument_bytes(ok) == [640 * 512 * 2, 640, 640, 1024, 1024, 640 * 512 * 2]
    with pytest.raises(H.AfirHipError, match="cover|tile|beyond"):     # halves do not add up
        r.argument_bytes(H.pack_tiling(640, 512, 320, 300, 512, 512, 640, 512))
    with pytest.raises(H.AfirHipError, match="runs past"):             # scale shorter than N
        r.argument_bytes(H.pack_tiling(640, 512, 320, 320, 100, 512, 640, 512))
    with pytest.raises(H.AfirHipError, match="tiling data must be"):
        r.argument_bytes(b"\0" * 8)
    r.close()
    g = H.Region(RC.RELU_COLGATHER_ADD)
    with pytest.raises(H.AfirHipError, match="does not match the output"):
        g.argument_bytes(H.pack_tiling(16, 640, 100, 128, 16, 128))
    with pytest.raises(H.AfirHipError, match="argument 2 runs past"):
        g.argument_bytes(H.pack_tiling(16, 640, 128, 100, 16, 128))
    g.close()


@pytest.mark.parametrize("bad,why", [
    ("", "header"),
    (RC.HEADER + "arg out f32 2\n", "no segment"),
    (RC.HEADER + "arg in f32 2\narg out f32 2\nsegment 2\n size arg0.0 arg0.1\n push arg0 d0 d1\n add\n store\nend\n",
     "fewer than two"),
    (RC.HEADER + "arg in f32 2\narg out f32 2\nsegment 2\n size arg0.0 arg0.1\n push arg0 d0 d1\nend\n", "end with 'store'"),
    (RC.HEADER + "arg in f32 2\narg out f32 2\nsegment 2\n size arg0.0 arg0.1\n push arg0 d0 d5\n store\nend\n",
     "missing iteration dim"),
    (RC.HEADER + "arg in f32 2\narg in f32 1\narg out f32 2\nsegment 2\n size arg0.0 arg0.1\n push arg0 d0 g1:arg1\n store\nend\n",
     "index tensor must be"),
    (RC.HEADER + "arg in f32 2\narg out f32 2\nsegment 2\n size arg0.0 arg0.1\n push arg0 d0 d1\n frobnicate\n store\nend\n",
     "unknown operation"),
    (RC.HEADER + "arg in f32 2\narg out f32 2\nsegment 2\n size arg0.0 arg0.1\n" + " push arg0 d0 d1\n" * 5 + " store\nend\n",
     "more than 4 live"),
    (RC.HEADER + "arg in f32 2\narg out f32 2\nsegment 2\n size arg0.0 arg0.1\n push arg0 d0 d1\n reduce sum\n store\nend\n",
     "output rank"),
    (RC.INT_ADD_I32.replace(" add\n", " div\n"), "'div' is not available in an integer region"),
    (RC.INT_ADD_I32.replace(" add\n", " add\n leaky 0.1\n"), "'leaky' is not available in an integer region"),
    (RC.INT_ADD_I32.replace(" add\n", " add\n reduce sum\n").replace("arg out i32 2", "arg out i32 1"),
     "'reduce sum' is not available in an integer region"),
    (RC.INT_ADD_I32.replace("arg in i32 2\narg in i32 2", "arg in i32 2\narg in f32 2"), "reads i16 / i32 tensors only"),
    (RC.INT_ADD_I32.replace(" add\n", " add\n const 0.5\n mul\n"), "must be a 32-bit integer"),
    (RC.C1_ADD_MUL.replace("arg in f32 2", "arg in i32 2", 1), "pushed tensors must be"),
])
def test_library_rejects_malformed_programs(H, bad, why):
    with pytest.raises(H.AfirHipError, match=why):
        H.Region(bad)


def test_mean_tail_is_pinned_by_exact_cases():
    """What follows 'reduce sum' works on the float32 sum.  Small integers make the sum exact
    and a power-of-two N makes the division exact, so the mean is fixed by the mathematics:
    it must equal the float64 mean rounded once to f16."""
    rng = np.random.default_rng(3)
    for m, n in ((5, 512), (64, 1024), (3, 8)):
        a = rng.integers(-8, 9, (m,)).astype(np.float16)
        b = rng.integers(-8, 9, (m, n)).astype(np.float16)
        got = RO.evaluate(RC.MEAN_ROWBIAS, [a, b])
        want = ((a.astype(np.float64)[:, None] + b.astype(np.float64)).sum(axis=1) / n).astype(np.float16)
        assert got.dtype == np.float16 and got.tobytes() == want.tobytes()
    # N that f16 cannot hold exactly: the IR converts the extent to f16 first (sitofp ... to f16),
    # 2049 becomes 2048
    a = np.zeros((2,), np.float16)
    b = np.ones((2, 2049), np.float16)
    assert RO.evaluate(RC.MEAN_ROWBIAS, [a, b]).tolist() == [np.float16(2049 / 2048)] * 2
    # ... and the sum: the IR keeps it in an f16 tensor, where 2049 is 2048 as well ('cast f16');
    # a program without that rounding divides the float32 sum
    assert RO.evaluate(RC.MEAN_ROWBIAS.replace("const arg1.1 f16", "const arg1.1"), [a, b]).tolist() == [1 - 2.0 ** -11] * 2
    plain = RC.MEAN_ROWBIAS.replace("  cast f16\n", "").replace("const arg1.1 f16", "const arg1.1")
    assert RO.evaluate(plain, [a, b]).tolist() == [1.0, 1.0]
    # a sum beyond the f16 range is infinite in that tensor, and so is the mean
    b = np.full((2, 2048), 40.0, np.float16)
    assert np.isinf(RO.evaluate(RC.MEAN_ROWBIAS, [a, b])).all()
    assert RO.evaluate(RC.MEAN_ROWBIAS.replace("  cast f16\n", ""), [a, b]).tolist() == [40.0, 40.0]


def test_mean_against_the_reference_written_sum_vector():
    """The reference's golden script writes the row SUMS of its example (as f16), which is the
    tensor the mean graph's division reads: the mean is that vector divided by N, exactly."""
    from tests import golden_cases as GC
    z = GC.load()
    a, b, sums = (np.ascontiguousarray(z["broadcast-add-reduce/" + k]) for k in ("input_a", "input_b", "output_c"))
    got = RO.evaluate(RC.MEAN_ROWBIAS, [a, b])
    assert got.tobytes() == RC.mean_rowbias_f16(a, b).tobytes()
    twice = (sums.astype(np.float32) / np.float32(b.shape[1])).astype(np.float16)
    assert got.tobytes() == twice.tobytes()


def test_reduce_tail_chain_matches_its_closed_form():
    text, inputs, want = RC.case_reduce_tail_chain()
    assert RO.evaluate(text, inputs).tobytes() == want.tobytes()


def test_matmul_layout_flags_against_numpy():
    """'ta' / 'tb' and the batched rank-3 form against numpy on the operands put back in the
    plain layout (float32 product of the widened operands, as the reference's golden computes it,
    examples/matmul-add-leakyrelu/gen_data.py:33)."""
    rng = np.random.default_rng(5)
    m, k, n, nb = 5, 7, 3, 4
    a = rng.standard_normal((m, k)).astype(np.float16)
    b = rng.standard_normal((k, n)).astype(np.float16)
    want = a.astype(np.float32) @ b.astype(np.float32)
    head = RC.HEADER + "arg in f16 2\narg in f16 2\narg out f32 2\nsegment 2\n size arg2.0 arg2.1\n outoff 0\n"
    for flags, aa, bb in (("", a, b), (" ta", a.T.copy(), b), (" tb", a, b.T.copy()), (" ta tb", a.T.copy(), b.T.copy())):
        got = RO.evaluate(head + f" matmul arg0 arg1{flags}\n store\nend\n", [aa, bb], out_shape=(m, n))
        assert got.dtype == np.float32 and np.array_equal(got, want), flags
    a3 = rng.standard_normal((nb, m, k)).astype(np.float16)
    b3 = rng.standard_normal((nb, n, k)).astype(np.float16)
    want3 = np.stack([a3[i].astype(np.float32) @ b3[i].astype(np.float32).T for i in range(nb)])
    prog = (RC.HEADER + "arg in f16 3\narg in f16 3\narg out f32 3\nsegment 3\n size arg2.0 arg2.1 arg2.2\n outoff 0\n"
            " matmul arg0 arg1 tb\n store\nend\n")
    got = RO.evaluate(prog, [a3, b3], out_shape=(nb, m, n))
    assert np.array_equal(got, want3)


def test_cast_is_the_rounding_of_the_storage_types():
    """'cast f16' / 'cast bf16' against numpy's float16 conversion and the bf16 bit formula the
    comparator decodes with (round to nearest even, overflow to infinity, NaN stays NaN), value
    by value on the corner cases: ties, the f16 overflow threshold, subnormals, zeros of both signs."""
    prog = RC.HEADER + "arg in f32 1\narg out f32 1\nsegment 1\n size arg0.0\n outoff 0\n push arg0 d0\n cast %s\n store\nend\n"
    x = np.array([0.0, -0.0, 1.0, 1.0 + 2.0 ** -11, 1.0 + 3 * 2.0 ** -11, 1.0 + 2.0 ** -10, 2049.0, 2051.0, 65504.0, 65519.99,
                  65520.0, -65520.0, 1e9, 6e-8, 2.9802322e-8, 2.99e-8, 5.9604645e-8, -1e-10, np.inf, -np.inf, np.nan,
                  1.0 + 2.0 ** -8, 1.0 + 3 * 2.0 ** -8, 3.4e38, 1.0 + 2.0 ** -7 + 2.0 ** -20], np.float32)
    got = RO.evaluate(prog % "f16", [x])
    by_hand = np.array([0.0, -0.0, 1.0, 1.0, 1.0 + 2.0 ** -9, 1.0 + 2.0 ** -10, 2048.0, 2052.0, 65504.0, 65504.0,
                        np.inf, -np.inf, np.inf, 2.0 ** -24, 0.0, 2.0 ** -24, 2.0 ** -24, -0.0, np.inf, -np.inf, np.nan,
                        1.0 + 2.0 ** -8, 1.0 + 3 * 2.0 ** -8, np.inf, 1.0 + 2.0 ** -7], np.float32)
    assert np.array_equal(got, by_hand, equal_nan=True) and np.signbit(got[1]) and np.signbit(got[17])
    with np.errstate(over="ignore"):
        assert np.array_equal(got, x.astype(np.float16).astype(np.float32), equal_nan=True)
    got = RO.evaluate(prog % "bf16", [x])
    by_hand_bf16 = {1.0 + 2.0 ** -8: 1.0, 1.0 + 3 * 2.0 ** -8: 1.0 + 2.0 ** -6, 1.0 + 2.0 ** -7 + 2.0 ** -20: 1.0 + 2.0 ** -7,
                    65504.0: 65536.0, 3.4e38: np.inf, 2049.0: 2048.0}
    for value, want in by_hand_bf16.items():
        assert got[np.flatnonzero(x == np.float32(value))[0]] == np.float32(want), value
    u = x.view(np.uint32).astype(np.uint64)
    formula = (((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16).astype(np.uint32).view(np.float32)
    finite = ~np.isnan(x)
    assert np.array_equal(got[finite], formula[finite]) and np.isnan(got[~finite]).all()
    assert np.array_equal(RO.evaluate(prog % "f32", [x]), x, equal_nan=True)
    rng = np.random.default_rng(0)
    y = rng.standard_normal(100000).astype(np.float32) * np.float32(1000)
    assert np.array_equal(RO.evaluate(prog % "f16", [y]), y.astype(np.float16).astype(np.float32))
