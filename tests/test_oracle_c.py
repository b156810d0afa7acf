"""Cross-checks of the C restatement against the numpy oracle.  CPU only."""
import numpy as np

from oracle import afir_oracle as O
from oracle import c_oracle as C


def test_f16_conversions_all_patterns():
    L = C.lib()
    allh = np.arange(65536, dtype=np.uint16)
    want = allh.view(np.float16).astype(np.float32)
    got = np.array([L.oracle_f16_to_f32(int(h)) for h in allh], np.float32)
    ok = ~np.isnan(want)
    assert np.array_equal(got[ok], want[ok])
    assert np.isnan(got[~ok]).all()
    # f32 -> f16 on every f16 value, every midpoint, and random floats
    r = np.random.default_rng(1)
    vals = np.concatenate([
        want[ok],
        ((want[ok][:-1].astype(np.float64) + want[ok][1:]) / 2).astype(np.float32),
        (r.standard_normal(20000) * 10.0 ** r.integers(-9, 6, 20000)).astype(np.float32),
        np.array([65504, 65519.99, 65520, 1e-8, 2.98e-8, 2.99e-8, 6e-8], np.float32),
    ])
    vals = vals[np.isfinite(vals)]
    with np.errstate(over="ignore"):
        want16 = vals.astype(np.float16).view(np.uint16)
    got16 = np.array([L.oracle_f32_to_f16(float(v)) for v in vals], np.uint16)
    assert np.array_equal(got16, want16)


def test_bf16_conversions():
    L = C.lib()
    r = np.random.default_rng(2)
    x = (r.standard_normal(20000) * 10.0 ** r.integers(-20, 20, 20000)).astype(np.float32)
    want = O.f32_to_bf16_bits(x)
    got = np.array([L.oracle_f32_to_bf16(float(v)) for v in x], np.uint16)
    assert np.array_equal(got, want)
    assert L.oracle_bf16_to_f32(0x3F80) == 1.0


def test_c1_bit_exact():
    a, b = O.gen_c1((257, 129))
    assert C.add_mul_f32(a, b).tobytes() == O.golden_c1(a, b).tobytes()


def test_c2_reproduces_numpy_pairwise_order():
    for m, n in [(33, 4096), (7, 5), (16, 128), (9, 129), (5, 1000), (3, 8192), (4, 300)]:
        x, bias = O.gen_c2(m, n)
        assert C.bcast_add_rowsum_f32(x, bias).tobytes() == \
            O.golden_c2(x, bias).tobytes(), (m, n)


def test_c3_bit_exact():
    x, c = O.gen_c3(3, 70, 36)
    assert C.relu_bcast_add_transpose_f16(x, c).tobytes() == \
        O.golden_c3(x, c).tobytes()


def test_c4_bit_exact():
    table, idx, scale, shift = O.gen_c4(1000, 136, 513)
    idx[:3] = [0, 999, 999]
    assert C.gather_scale_shift_f16(table, idx, scale, shift).tobytes() == \
        O.golden_c4(table, idx, scale, shift).tobytes()


def test_c4_rejects_out_of_range():
    table, idx, scale, shift = O.gen_c4(16, 8, 4)
    idx[1] = 16
    try:
        C.gather_scale_shift_f16(table, idx, scale, shift)
    except IndexError:
        return
    raise AssertionError("out-of-range index accepted")


def test_c5_within_tolerance_of_numpy():
    a, b, bias = O.gen_c5(48, 1024, 80)
    got = C.matmul_bias_leakyrelu_bf16(a, b, bias, 0.01)
    want = O.golden_c5(a, b, bias, 0.01)
    r = O.compare_outputs([(got, "bf16")], [(want, "bf16")], 1e-5, 1e-2)
    assert r["passed"], r
    assert (got == want).mean() > 0.98


def test_c5_integer_inputs_exact():
    r = np.random.default_rng(42)
    A = r.integers(-10, 10, (32, 256)).astype(np.float32)
    B = r.integers(-10, 10, (256, 40)).astype(np.float32)
    bias = r.integers(1, 10, (40,)).astype(np.float32)
    args = [O.f32_to_bf16_bits(v) for v in (A, B, bias)]
    assert np.array_equal(C.matmul_bias_leakyrelu_bf16(*args, 0.01),
                          O.golden_c5(*args, 0.01))


def test_compare_matches_numpy_comparator():
    r = np.random.default_rng(3)
    e = r.standard_normal(5000).astype(np.float16)
    a = (e.astype(np.float32) * (1 + 2e-3 * r.standard_normal(5000))).astype(np.float16)
    for atol, rtol in [(0, 0), (1e-3, 1e-3), (1e-2, 1e-2)]:
        c = C.compare(a, e, "f16", atol, rtol)
        p = O.compare_outputs([(a, "f16")], [(e, "f16")], atol, rtol)
        assert c["mismatches"] == p["mismatches"]
        assert abs(c["max_abs_diff"] - p["max_abs_diff"]) < 1e-12
        assert c["passed"] == p["passed"]
