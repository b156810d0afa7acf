"""Pins for the numpy oracle: golden vectors and known answers held by the
reference's own tests, closed forms and brute force.  CPU only."""
import struct

import numpy as np
import pytest

from oracle import afir_oracle as O


def _f32(x):
    return struct.unpack("<f", struct.pack("<f", x))[0]


# ---- C1: add -> mul chain -------------------------------------------------

def test_c1_bruteforce_and_special_cases():
    a, b = O.gen_c1((4, 4))          # README example is a 4x4 chain
    out = O.golden_c1(a, b)
    for i in range(4):
        for j in range(4):
            s = _f32(float(a[i, j]) + float(b[i, j]))
            assert out[i, j] == np.float32(_f32(s * float(b[i, j])))
    z = np.zeros_like(a)
    assert np.array_equal(O.golden_c1(a, z), z * a)          # b = 0
    one = np.ones_like(a)
    assert np.array_equal(O.golden_c1(a, one), a + one)       # b = 1
    assert np.array_equal(np.abs(O.golden_c1(a, -a)), z)      # a = -b


def test_c1_is_two_roundings_not_one():
    # (a+b)*b with one rounding (f64 then cast) differs somewhere: the golden
    # must round after the add.
    a, b = O.gen_c1((256, 256))
    two = O.golden_c1(a, b)
    one = ((a.astype(np.float64) + b) * b).astype(np.float32)
    assert (two != one).any()
    assert np.allclose(two, one, rtol=1e-6, atol=1e-7)


# ---- shape rules pinned by the reference's lit tests ----------------------

def test_broadcast_shape_rules():
    assert O.broadcast_shape((4, 1, 31), (1, 30, 1)) == (4, 30, 31)
    assert O.broadcast_shape((4096,), (8192, 4096)) == (8192, 4096)
    with pytest.raises(ValueError):
        O.broadcast_shape((4, 3), (4, 5))


def test_reduce_shape_rules():
    assert O.reduce_shape((4, 5), 0) == (5,)
    assert O.reduce_shape((4, 5), 1) == (4,)
    with pytest.raises(ValueError):
        O.reduce_shape((4, 5), 2)


# ---- C2: broadcast add + row sum -----------------------------------------

def test_c2_invariant_and_exact_cases():
    x, bias = O.gen_c2(64, 512)
    y = O.golden_c2(x, bias)
    ref = x.astype(np.float64).sum(axis=1) + bias.astype(np.float64).sum()
    scale = np.abs(x.astype(np.float64) + bias).sum(axis=1)
    assert np.all(np.abs(y - ref) <= 1e-6 * scale)
    ones = np.ones((8, 4096), np.float32)
    assert np.array_equal(O.golden_c2(ones, np.zeros(4096, np.float32)),
                          np.full(8, 4096, np.float32))
    onehot = np.zeros((4, 128), np.float32)
    onehot[np.arange(4), [0, 5, 77, 127]] = 3.0
    assert np.array_equal(O.golden_c2(onehot, np.ones(128, np.float32)),
                          np.full(4, 131, np.float32))


def test_c2_bias_is_per_column():
    x = np.zeros((3, 4), np.float32)
    bias = np.array([1, 2, 4, 8], np.float32)
    assert np.array_equal(O.golden_c2(x, bias), np.full(3, 15, np.float32))


def test_ref_shaped_reduce_rowbias():
    a = np.array([1, 2], np.float16)
    b = np.ones((2, 16), np.float16)
    assert np.array_equal(O.reduce_rowbias_f16(a, b),
                          np.array([32, 48], np.float16))


# ---- relu / broadcast add microcases (closed forms) -----------------------

def test_relu_microcase():
    x = np.array([-8.0 + 16.0 * i / 639.0 for i in range(640)], np.float16)
    exp = np.array([max(-8.0 + 16.0 * i / 639.0, 0.0) for i in range(640)],
                   np.float16)
    assert np.array_equal(O.op_relu(x.astype(np.float32)).astype(np.float16), exp)


def test_broadcast_add_microcase():
    base = np.array([i / 64.0 for i in range(640)], np.float16).reshape(1, 640)
    bias = np.array([i / 128.0 for i in range(1280)], np.float16).reshape(2, 640)
    exp = np.array([(i % 640) / 64.0 + i / 128.0 for i in range(1280)],
                   np.float16).reshape(2, 640)
    got = O.op_add(base.astype(np.float32), bias.astype(np.float32))
    assert O.broadcast_shape(base.shape, bias.shape) == (2, 640)
    # inputs are f16-rounded before the add in the kernel; the microcase's
    # expectation rounds the exact sum: equal wherever both are representable
    assert np.allclose(got.astype(np.float16).astype(np.float32),
                       exp.astype(np.float32), rtol=2e-3)


def test_leaky_relu_forms_agree():
    x = np.linspace(-4, 4, 1001, dtype=np.float32)
    for alpha in (0.0, 0.001, 0.01, 1.0):
        usual = np.where(x >= 0, x, x * np.float32(alpha))
        assert np.array_equal(O.op_leaky_relu(x, alpha), usual)


# ---- C3: relu + bias + transpose -----------------------------------------

def test_c3_bruteforce_and_involution():
    x, c = O.gen_c3(2, 3, 5)
    out = O.golden_c3(x, c)
    assert out.shape == (2, 5, 3)
    for b in range(2):
        for i in range(3):
            for j in range(5):
                v = np.float32(max(float(x[b, i, j]), 0.0)) + np.float32(c[j])
                assert out[b, j, i] == np.float16(v)
    zero = np.zeros(5, np.float16)
    pos = np.abs(x)
    assert np.array_equal(
        O.golden_c3(O.golden_c3(pos, zero), np.zeros(3, np.float16)), pos)


def test_ref_shaped_relu_col_add():
    d0 = np.array([[-1.0], [2.0]], np.float16)
    d1 = np.ones((3, 2), np.float16)
    assert np.array_equal(O.relu_col_add_f16(d0, d1),
                          np.tile(np.array([1, 3], np.float16), (3, 1)))


# ---- C4: gather * scale + shift ------------------------------------------

def test_c4_identity_and_boundaries():
    table, idx, scale, shift = O.gen_c4(512, 64, 256)
    idx[:4] = [0, 511, 511, 0]                     # boundary + repeated
    one = np.ones(64, np.float16)
    zero = np.zeros(64, np.float16)
    out = O.golden_c4(table, idx, one, zero)
    assert out.tobytes() == table[idx].tobytes()
    out = O.golden_c4(table, idx, scale, shift)
    r, j = 7, 13
    v = np.float32(table[idx[r], j]) * np.float32(scale[j]) + np.float32(shift[j])
    assert out[r, j] == np.float16(v)


def test_c4_fused_equals_unfused():
    # f16*f16 is exact in f32, so a fused multiply-add rounds identically
    table, idx, scale, shift = O.gen_c4(256, 128, 128)
    g = table[idx].astype(np.float64)
    fused = (g * scale.astype(np.float64) + shift.astype(np.float64)) \
        .astype(np.float32).astype(np.float16)
    # double rounding f64->f32->f16 can differ from the golden only at
    # f32 ties, which cannot occur for these magnitudes: require equality
    assert np.array_equal(fused, O.golden_c4(table, idx, scale, shift))


def test_ref_shaped_column_gather():
    data = np.arange(12, dtype=np.float16).reshape(2, 6) - 4
    idx = np.array([5, 0], np.int64)
    bias = np.array([0.5, 1.0], np.float16)
    exp = np.array([[1.5, 1.0], [7.5, 3.0]], np.float16)
    assert np.array_equal(O.relu_colgather_add_f16(data, idx, bias), exp)


# ---- C5: matmul + bias + leaky relu --------------------------------------

def test_c5_small_integer_known_answer():
    # the reference's trick: small integers make f32 accumulation exact
    r = np.random.default_rng(42)
    M, K, N = 128, 256, 128
    A = r.integers(-10, 10, (M, K))
    B = r.integers(-10, 10, (K, N))
    bias = r.integers(1, 10, (N,))
    exact = A.astype(object) @ B.astype(object) + bias.astype(object)   # Python ints
    a_bits = O.f32_to_bf16_bits(A.astype(np.float32))
    b_bits = O.f32_to_bf16_bits(B.astype(np.float32))
    bias_bits = O.f32_to_bf16_bits(bias.astype(np.float32))
    assert np.array_equal(O.bf16_bits_to_f32(a_bits), A.astype(np.float32))
    got = O.bf16_bits_to_f32(O.golden_c5(a_bits, b_bits, bias_bits, 0.01))
    exact_f = np.array(exact, dtype=np.float64)
    want = np.where(exact_f >= 0, exact_f, exact_f * np.float64(np.float32(0.01)))
    # output is rounded to bf16 (8 significant bits): half an ulp is 2^-9 relative
    assert np.all(np.abs(got - want) <= np.abs(want) * 2.0 ** -8 + 1e-30)
    # f16 reference-shaped variant is exact
    E = O.matmul_bias_leakyrelu_f16(A.astype(np.float16), B.astype(np.float16),
                                    bias.astype(np.float32), 0.001)
    want32 = np.where(exact_f >= 0, exact_f,
                      (exact_f.astype(np.float32) * np.float32(0.001)))
    assert np.array_equal(E, want32.astype(np.float32))


def test_c5_matches_torch_f32_matmul():
    import torch
    a, b, bias = O.gen_c5(64, 512, 96)
    got = O.bf16_bits_to_f32(O.golden_c5(a, b, bias))
    ta = torch.from_numpy(O.bf16_bits_to_f32(a))
    tb = torch.from_numpy(O.bf16_bits_to_f32(b))
    acc = ta @ tb + torch.from_numpy(O.bf16_bits_to_f32(bias))
    want = torch.nn.functional.leaky_relu(acc, 0.01).to(torch.bfloat16).float().numpy()
    assert np.allclose(got, want, rtol=1e-2, atol=1e-6)
    assert (got == want).mean() > 0.99


def test_bf16_rne():
    cases = {0x3F800000: 0x3F80, 0x3F808000: 0x3F80, 0x3F818000: 0x3F82,
             0x3F808001: 0x3F81, 0x7F800000: 0x7F80, 0xBF800000: 0xBF80}
    for u, want in cases.items():
        f = np.array([u], np.uint32).view(np.float32)
        assert int(O.f32_to_bf16_bits(f)[0]) == want
    import torch
    x = np.random.default_rng(0).standard_normal(10000).astype(np.float32)
    t = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(O.f32_to_bf16_bits(x), t)


# ---- comparator -----------------------------------------------------------

def test_comparator_reference_cases():
    a = np.array([1.0, 2.0], np.float32)
    r = O.compare_outputs([(a, "f32")], [(a.copy(), "f32")], 0.0, 0.0)
    assert r["passed"] and r["max_abs_diff"] == 0.0 and r["mean_abs_diff"] == 0.0
    assert r["error_message"] == ""
    b = np.array([1.0, 2.25], np.float32)
    r = O.compare_outputs([(b, "f32")], [(a, "f32")], 1e-4, 1e-4)
    assert not r["passed"] and r["max_abs_diff"] > 0 and r["mean_abs_diff"] > 0
    assert r["error_message"]
    with pytest.raises(O.StructuralMismatch):
        O.compare_outputs([(a, "f32")], [], 0.0, 0.0)
    with pytest.raises(O.StructuralMismatch):
        O.compare_outputs([(a, "f32")], [(a.reshape(1, 2), "f32")], 0.0, 0.0)
    with pytest.raises(O.StructuralMismatch):
        O.compare_outputs([(a, "f32")],
                          [(np.array([1, 2], np.int32), "i32")], 0.0, 0.0)


def test_comparator_is_nan_blind_and_nonfinite_mismatches_is_not():
    """The reference's `diff > atol + rtol*|e|` is false for NaN, so its comparator passes
    a NaN where the golden is finite; the parity checks count those separately."""
    want = np.array([1.0, -2.0, np.inf, -np.inf, np.nan, 0.0], np.float32)
    got = np.array([np.nan, -2.0, np.inf, np.inf, np.nan, np.inf], np.float32)
    r = O.compare_outputs([(got, "f32")], [(want, "f32")], 1e-5, 1e-2)
    assert r["mismatches"] == 1          # only the finite-vs-inf element at the end
    assert O.nonfinite_mismatches(got, want, "f32") == 3   # NaN vs 1, +inf vs -inf, inf vs 0
    assert O.nonfinite_mismatches(want, want, "f32") == 0
    # bf16 bits: 0x7fc0 NaN, 0x7f80 +inf, 0x3f80 1.0
    gb = np.array([0x7fc0, 0x7f80, 0x3f80], np.uint16)
    wb = np.array([0x3f80, 0x7f80, 0x3f80], np.uint16)
    assert O.compare_outputs([(gb, "bf16")], [(wb, "bf16")], 1e-5, 1e-2)["passed"]
    assert O.nonfinite_mismatches(gb, wb, "bf16") == 1


def test_comparator_decode_bits():
    assert O.comparator_decode(np.array([0x3C00], np.uint16), "f16")[0] == 1.0
    assert O.comparator_decode(np.array([0x4000], np.uint16), "f16")[0] == 2.0
    assert O.comparator_decode(np.array([0x3F80], np.uint16), "bf16")[0] == 1.0
    allh = np.arange(65536, dtype=np.uint16)
    exp = (allh >> 10) & 0x1F
    normal = (exp != 0) & (exp != 31)
    assert np.array_equal(O.comparator_decode(allh, "f16")[normal],
                          allh.view(np.float16).astype(np.float32)[normal])


# ---- tiling bytes ----------------------------------------------------------

SIX = [("TB_M", "int64"), ("TB_N", "int64"), ("dim_arg0_0", "int64"),
       ("dim_arg1_1", "int64"), ("dim_arg0_1", "int64"), ("dim_arg1_0", "int64")]


def test_tiling_pack_known_answers():
    b = O.pack_tiling(SIX, [("TB_M", 16), ("TB_N", 16), ("dim_arg0_0", 64),
                            ("dim_arg1_1", 64), ("dim_arg0_1", 64),
                            ("dim_arg1_0", 64)])
    assert len(b) == 48
    assert struct.unpack("<q", b[:8])[0] == 16
    assert struct.unpack("<q", b[40:48])[0] == 64
    mixed = [("A", "int64"), ("B", "int32"), ("C", "int64")]
    b = O.pack_tiling(mixed, [("A", 1), ("B", 2), ("C", 3)])
    assert len(b) == 20
    assert struct.unpack("<qiq", b) == (1, 2, 3)


def test_tiling_pack_errors():
    with pytest.raises(O.TilingError, match="count mismatch"):
        O.pack_tiling(SIX, [("TB_M", 16), ("TB_N", 16)])
    bad = [("WRONG", 16)] + [(n, 64) for n, _ in SIX[1:]]
    with pytest.raises(O.TilingError, match="name mismatch.*WRONG.*TB_M"):
        O.pack_tiling(SIX, bad)
    with pytest.raises(O.TilingError, match="missing field"):
        O.pack_tiling_named(SIX, "TB_M=16")
    b = O.pack_tiling_named(
        SIX, "dim_arg1_0=640,TB_M=16,TB_N=16,dim_arg0_0=640,dim_arg1_1=512,dim_arg0_1=1")
    assert struct.unpack("<6q", b) == (16, 16, 640, 512, 1, 640)


def test_tiling_schema_json(tmp_path):
    p = tmp_path / "t.json"
    p.write_text('{"tiling_params": [{"name": "A"}, {"name": "B", "type": "int32"}]}')
    assert O.load_tiling_schema(p) == [("A", "int64"), ("B", "int32")]
    p.write_text("{ not valid json")
    with pytest.raises(Exception):
        O.load_tiling_schema(p)


# ---- npy -------------------------------------------------------------------

def _write_npy(path, descr, shape, payload):
    d = "{'descr': '%s', 'fortran_order': False, 'shape': (%s,), }" % (
        descr, ",".join(str(s) for s in shape))
    total = 10 + len(d) + 1
    d += " " * ((64 - total % 64) % 64) + "\n"
    with open(path, "wb") as f:
        f.write(b"\x93NUMPY\x01\x00" + struct.pack("<H", len(d)) + d.encode() + payload)


def test_npy_known_answers(tmp_path):
    cases = [
        ("<f2", np.array([0x3C00, 0x4000, 0], np.uint16), "f16"),
        ("<V2", np.array([0x3F80, 0x4000, 0], np.uint16), "bf16"),
        ("<f4", np.array([1, 2, 3, 4], np.float32), "f32"),
        ("|i1", np.array([1, -2, 127, -128], np.int8), "i8"),
        ("<i4", np.array([100, -200, 0, 2147483647], np.int32), "i32"),
        ("<i8", np.array([1000000, -2000000, 0], np.int64), "i64"),
    ]
    for descr, arr, dt in cases:
        p = tmp_path / "in.npy"
        _write_npy(p, descr, arr.shape, arr.tobytes())
        got, gdt = O.load_npy(p)
        assert gdt == dt and got.shape == arr.shape
        assert got.tobytes() == arr.tobytes()
        q = tmp_path / "out.npy"
        O.save_npy(q, got, gdt)
        raw = open(q, "rb").read()
        hlen = struct.unpack("<H", raw[8:10])[0]
        assert (10 + hlen) % 64 == 0 and raw[10 + hlen - 1:10 + hlen] == b"\n"
        back, bdt = O.load_npy(q)
        assert bdt == dt and back.tobytes() == arr.tobytes()
        viaNumpy = np.load(q)
        assert viaNumpy.tobytes() == arr.tobytes()
        if dt == "bf16":
            assert viaNumpy.dtype.str == "|V2" or viaNumpy.dtype.str == "<V2"


def test_npy_rejections(tmp_path):
    p = tmp_path / "f64.npy"
    _write_npy(p, "<f8", (2,), np.array([1.0, 2.0]).tobytes())
    with pytest.raises(O.NpyError, match="Unsupported dtype"):
        O.load_npy(p)
    with pytest.raises(O.NpyError, match="Cannot open"):
        O.load_npy(tmp_path / "missing.npy")
    p = tmp_path / "trunc.npy"
    _write_npy(p, "<f4", (3,), np.array([1.0], np.float32).tobytes())
    with pytest.raises(O.NpyError, match="Truncated"):
        O.load_npy(p)
    p = tmp_path / "bad.npy"
    p.write_bytes(b"hello world, not numpy")
    with pytest.raises(O.NpyError, match="Not a .npy"):
        O.load_npy(p)


def test_npy_shapes(tmp_path):
    for shape in [(3,), (2, 3), (2, 3, 4)]:
        arr = np.arange(np.prod(shape), dtype=np.float32).reshape(shape)
        p = tmp_path / "s.npy"
        O.save_npy(p, arr, "f32")
        assert np.array_equal(np.load(p), arr)
        got, _ = O.load_npy(p)
        assert got.shape == shape


def test_algorithmic_bytes_match_published_table():
    assert O.algorithmic_bytes("c1", m=4096, n=4096) == 201326592
    assert O.algorithmic_bytes("c2", m=8192, n=4096) == 134266880
    assert O.algorithmic_bytes("c3", b=64, m=1024, n=512) == 134218752
    assert O.algorithmic_bytes("c4", nidx=32768, dim=1024) == 134352896
    assert O.algorithmic_flops_c5(8192, 8192, 8192) == 1099511627776
