"""afir-translate -mlir-to-hip: MLIR text -> region program.  Each translated
program is evaluated with the region oracle and must reproduce the closed-form
golden of the graph it came from.  CPU only."""
import json
import os
import subprocess

import numpy as np
import pytest

from oracle import afir_oracle as O
from oracle import region_oracle as RO
from tests import mlir_cases as MC
from tests import region_cases as RC

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TR = os.path.join(ROOT, "ascend-mlir_amd", "bin", "afir-translate")
REF_EXAMPLES = "/root/reference/examples"


def translate(text, *extra):
    p = subprocess.run([TR, "-mlir-to-hip", "-", *extra], input=text, capture_output=True, text=True)
    return p.returncode, p.stdout, p.stderr


def program_of(text):
    rc, out, err = translate(text)
    assert rc == 0, err
    return out


CASES = [
    (MC.ROW_BIAS_REDUCE, RC.case_reduce_rowbias, "rowbias_reduce"),
    (MC.RELU_COLUMN_ADD, RC.case_relu_col_add, "relu_column_add"),
    (MC.RELU_GATHER_COLUMNS_ADD, RC.case_relu_colgather_add, "relu_gather_columns_add"),
    (MC.TWO_CHAINS_CONCAT, RC.case_add_broadcast_concat, "two_chains_concat"),
    (MC.SPLIT_HALVES, RC.case_split_relu_brc_add_mul, "split_halves"),
    (MC.C1_AFIR, RC.case_c1, "add_mul"),
    (MC.C2_LINALG, RC.case_c2, "bcast_add_rowsum"),
    (MC.C3_LINALG, RC.case_c3, "relu_bcast_transpose"),
    (MC.C4_LINALG, RC.case_c4, "gather_scale_shift"),
]


@pytest.mark.parametrize("mlir,case,name", CASES, ids=[c[2] for c in CASES])
def test_translated_program_reproduces_the_golden(mlir, case, name):
    out = program_of(mlir)
    assert out.splitlines()[0] == f"# kernel {name}"
    _, inputs, want = case()
    got = RO.evaluate(out, inputs)
    assert got.dtype == want.dtype and got.tobytes() == want.tobytes()


def test_benchmark_graphs_route_to_the_hand_tuned_kernels(pkg):
    from ascend_mlir_amd import hip_kernels as H
    H.load()
    for mlir, want in [(MC.C1_AFIR, "fused_add_mul"), (MC.C2_LINALG, "broadcast_add_reducesum"),
                       (MC.C3_LINALG, "relu_broadcast_add_transpose"), (MC.C4_LINALG, "gather_scale_shift"),
                       (MC.MATMUL_BIAS_LEAKY_BF16, "matmul_add_leakyrelu"),
                       (MC.RELU_COLUMN_ADD, "fused_region"), (MC.SPLIT_HALVES, "fused_region")]:
        r = H.Region(program_of(mlir))
        assert r.kernel == want
        r.close()


def test_matmul_epilogue_kinds_none_and_bias_add(pkg):
    """The reference annotates matmul regions with the epilogue kinds None,
    BiasAdd and BiasAddLeakyRelu
    (lib/Conversion/MarkStructuredOps/AnnotateMixMatmulSemanticsPass.cpp:319-323);
    all three become a matmul program on the MFMA kernels."""
    from ascend_mlir_amd import hip_kernels as H
    for mlir, tail in ((MC.MATMUL_PLAIN_F16, ["matmul arg0 arg1", "store", "end"]),
                       (MC.MATMUL_BIAS_F16, ["matmul arg0 arg1", "push arg2 d1", "add", "store", "end"]),
                       (MC.MATMUL_PLAIN_BF16, ["matmul arg0 arg1", "store", "end"]),
                       (MC.MATMUL_BIAS_BF16, ["matmul arg0 arg1", "push arg2 d1", "add", "store", "end"]),
                       # the runtime's BiasAddRelu (include/Runtime/Mix/MatmulTilingTypes.h:13) and relu alone
                       (MC.MATMUL_BIAS_RELU_F16, ["matmul arg0 arg1", "push arg2 d1", "add", "relu", "store", "end"]),
                       (MC.MATMUL_BIAS_RELU_BF16, ["matmul arg0 arg1", "push arg2 d1", "add", "relu", "store", "end"]),
                       (MC.MATMUL_RELU_F16, ["matmul arg0 arg1", "relu", "store", "end"]),
                       (MC.MATMUL_RELU_BF16, ["matmul arg0 arg1", "relu", "store", "end"])):
        out = program_of(mlir)
        body = [l.strip() for l in out.splitlines() if l.strip() and not l.startswith("#")]
        assert body[-len(tail):] == tail, out
        r = H.Region(out)
        assert r.kernel == ("matmul_add_leakyrelu" if "bf16" in mlir else "matmul_add_leakyrelu_f16")
        r.close()
    # an epilogue outside the vocabulary is refused at registration
    odd = program_of(MC.MATMUL_BIAS_F16).replace("add\n", "mul\n")
    with pytest.raises(H.AfirHipError, match="other epilogues are not implemented"):
        H.Region(odd)


def test_matmul_epilogue_program_and_alpha():
    out = program_of(MC.MATMUL_BIAS_LEAKY_F16)
    body = [l for l in out.splitlines() if l and not l.startswith(("#", "afir-hip", "arg"))]
    assert body == ["segment 2", "size arg3.0 arg3.1", "outoff 0", "matmul arg0 arg1", "push arg2 d1",
                    "add", "leaky 0.00100000005", "store", "end"]
    assert [l for l in out.splitlines() if l.startswith("arg")] == [
        "arg in f16 2", "arg in f16 2", "arg in f32 1", "arg in f32 2", "arg out f32 2"]


def test_afir_broadcast_chain_matches_numpy():
    rng = np.random.default_rng(9)
    a = rng.uniform(-2, 2, (4, 1, 31)).astype(np.float32)
    b = rng.uniform(-2, 2, (1, 30, 1)).astype(np.float32)
    out = program_of(MC.AFIR_BROADCAST_CHAIN)
    got = RO.evaluate(out, [a, b])
    t = b - (a + b) * b
    want = np.maximum(t, t * np.float32(0.01)).astype(np.float32)
    assert got.shape == (4, 30, 31) and got.tobytes() == want.tobytes()     # 4x1x31 (+) 1x30x1 -> 4x30x31


def test_afir_div_relu_sum_matches_numpy():
    rng = np.random.default_rng(10)
    a = rng.uniform(-2, 2, (6, 40)).astype(np.float32)
    b = rng.uniform(0.5, 2, (40,)).astype(np.float32)
    got = RO.evaluate(program_of(MC.AFIR_DIV_RELU_SUM), [a, b])
    want = np.maximum(a / b[None, :], np.float32(0)).sum(axis=1, dtype=np.float32)
    assert got.shape == (6,) and got.tobytes() == want.tobytes()


def test_tiling_space_out(tmp_path):
    ts = tmp_path / "tiling_space.json"
    rc, out, err = translate(MC.RELU_GATHER_COLUMNS_ADD, "--tiling-space-out", str(ts))
    assert rc == 0, err
    d = json.loads(ts.read_text())
    assert d["kernel"] == "relu_gather_columns_add" and d["soc"] == "gfx950"
    assert [p["name"] for p in d["tiling_params"]] == [
        "dim_arg0_0", "dim_arg0_1", "dim_arg1_0", "dim_arg2_0", "dim_arg3_0", "dim_arg3_1"]
    assert all(p["type"] == "int64" for p in d["tiling_params"])


@pytest.mark.parametrize("text,why", [
    ("", "no func.func"),
    ("func.func @f(%a: tensor<4xf32>) -> tensor<4xf32> {\n %0 = afir.exp %a : tensor<4xf32> -> tensor<4xf32>\n return %0 : tensor<4xf32>\n}",
     "line 2: afir.exp has no HIP lowering"),
    ("func.func @f(%a: tensor<4xf32>) -> tensor<4xf32> {\n %0 = math.tanh %a : tensor<4xf32>\n return %0 : tensor<4xf32>\n}",
     "operation 'math.tanh' has no HIP lowering"),
    ("func.func @f(%a: tensor<4xf64>) -> tensor<4xf64> {\n return %a : tensor<4xf64>\n}", "unsupported element type 'f64'"),
    (MC.C3_LINALG.replace("affine_map<(d0, d1, d2) -> (d0, d1, d2)>],", "affine_map<(d0, d1, d2) -> (d0, d2, d1)>],"),
     "only an identity output map"),
    (MC.C2_LINALG.replace('["parallel", "reduction"]', '["reduction", "parallel"]'), "reduction over the last iteration dim"),
    (MC.C2_LINALG.replace("%v = arith.addf %a, %acc : f32", "%v = arith.mulf %a, %acc : f32"), "only a sum reduction"),
    (MC.C2_LINALG.replace("arith.constant 0.0 : f32", "arith.constant 1.0 : f32"), "zero-filled init"),
    (MC.TWO_CHAINS_CONCAT.replace("dim(0)", "dim(1)"), "along dim 0 only"),
    (MC.C1_AFIR.replace("return %1", "return %9"), "undefined value %9"),
    (MC.RELU_COLUMN_ADD.replace("(d0, d1) -> (d1, 0)", "(d0, d1) -> (d1 + 1, 0)"), "only dimensions and constants"),
    ("func.func @f(%a: tensor<4x8xf32>, %b: tensor<4x8xf32>) -> tensor<4x8xf32> {\n"
     " %0 = afir.add %a, %b : (tensor<8xf32>, tensor<4x8xf32>) -> tensor<4x8xf32>\n return %0 : tensor<4x8xf32>\n}",
     "line 2: afir.add: the type given for %a has another rank than the value"),
])
def test_unsupported_input_is_rejected_with_a_diagnostic(text, why):
    rc, out, err = translate(text)
    assert rc == 1 and why in err, err


def test_usage_errors():
    assert subprocess.run([TR]).returncode == 2
    assert subprocess.run([TR, "-mlir-to-cann", "x.mlir"], capture_output=True).returncode == 2
    assert subprocess.run([TR, "-mlir-to-hip", "/no/such/file.mlir"], capture_output=True).returncode == 2
    assert subprocess.run([TR, "--help"], capture_output=True).returncode == 0


# The reference's own example inputs, where the reference tree is present
# (it is not on the GPU box): read as text, translated, evaluated, compared
# with the closed-form golden of the example.
REF_CASES = [
    ("broadcast-add-reduce", RC.case_reduce_rowbias),
    ("relu-broadcast-transpose", RC.case_relu_col_add),
    ("gather-elementwise-fusion", RC.case_relu_colgather_add),
    ("add-broadcast-concat", RC.case_add_broadcast_concat),
    ("split-relu-brc-add-mul", RC.case_split_relu_brc_add_mul),
]


@pytest.mark.skipif(not os.path.isdir(REF_EXAMPLES), reason="reference tree not present")
@pytest.mark.parametrize("example,case", REF_CASES, ids=[c[0] for c in REF_CASES])
def test_reference_example_inputs_translate_and_evaluate(example, case):
    p = subprocess.run([TR, "-mlir-to-hip", os.path.join(REF_EXAMPLES, example, "step0_input.mlir")],
                       capture_output=True, text=True)
    assert p.returncode == 0, p.stderr
    _, inputs, want = case()
    assert RO.evaluate(p.stdout, inputs).tobytes() == want.tobytes()


def test_mean_is_a_sum_with_a_tail_on_the_row_sums():
    """Reduce followed by an elementwise generic on the sums (mean = sum / N): the extent
    reaches the body through arith.index_cast + arith.sitofp, outside any generic."""
    out = program_of(MC.ROW_BIAS_MEAN)
    body = [l.strip() for l in out.splitlines() if l.strip() and not l.startswith("#")]
    assert body[body.index("outoff 0") + 1:] == [
        "push arg0 d0", "push arg1 d0 d1", "add", "reduce sum", "cast f16", "const arg1.1 f16", "div", "store", "end"]
    _, inputs, want = RC.case_mean_rowbias(33, 96)
    assert RO.evaluate(out, inputs).tobytes() == want.tobytes()
    # c - sum, sum * c, max(sum, c): the sum as either operand where the operation allows it
    for expr, tail in (("arith.subf %nf, %x", ["neg", "const arg1.1 f16", "add"]),
                       ("arith.mulf %nf, %x", ["const arg1.1 f16", "mul"]),
                       ("arith.maximumf %x, %nf", ["const arg1.1 f16", "max"])):
        out = program_of(MC.ROW_BIAS_MEAN.replace("arith.divf %x, %nf", expr))
        body = [l.strip() for l in out.splitlines() if l.strip() and not l.startswith("#")]
        assert body[body.index("reduce sum") + 1:-2] == ["cast f16"] + tail, expr    # the sums are an f16 tensor
    bad = subprocess.run([TR, "-mlir-to-hip", "-"], input=MC.ROW_BIAS_MEAN.replace("arith.divf %x, %nf", "arith.divf %nf, %x"),
                         capture_output=True, text=True)
    assert bad.returncode != 0 and "divided by a reduced value" in bad.stderr


@pytest.mark.skipif(not os.path.isdir(REF_EXAMPLES), reason="reference tree not present")
def test_reference_mean_example_translates_unchanged():
    p = subprocess.run([TR, "-mlir-to-hip", os.path.join(REF_EXAMPLES, "broadcast-add-reduce", "step0_input_mean.mlir")],
                       capture_output=True, text=True)
    assert p.returncode == 0, p.stderr
    _, inputs, want = RC.case_mean_rowbias()
    assert RO.evaluate(p.stdout, inputs).tobytes() == want.tobytes()


def test_asc_graph_form_with_load_store_and_attribute_dictionaries():
    out = program_of(MC.ASC_GRAPH_FORM)
    body = [l.strip() for l in out.splitlines() if l.strip() and not l.startswith("#")]
    assert body[body.index("outoff 0") + 1:] == [
        "push arg0 d0 d1", "push arg1 0 d1", "add", "push arg0 d0 d1", "push arg1 0 d1", "add", "push arg1 0 d1",
        "mul", "sub", "store", "end"]
    rng = np.random.default_rng(4)
    x = rng.uniform(-2, 2, (12, 40)).astype(np.float32)
    y = rng.uniform(-2, 2, (1, 40)).astype(np.float32)
    s = x + y
    assert RO.evaluate(out, [x, y]).tobytes() == (s - s * y).astype(np.float32).tobytes()


@pytest.mark.skipif(not os.path.isfile("/root/reference/python/afir-to-ascir/asc_graph.afir"),
                    reason="reference tree not present")
def test_reference_asc_graph_file_translates():
    p = subprocess.run([TR, "-mlir-to-hip", "/root/reference/python/afir-to-ascir/asc_graph.afir"],
                       capture_output=True, text=True)
    assert p.returncode == 0, p.stderr
    assert "# kernel HashCopyAscGraph" in p.stdout and p.stdout.rstrip().endswith("mul\nsub\nstore\nend")


AFIR_LIT = "/root/reference/test/Dialect/AFIR/ops.mlir"


@pytest.mark.skipif(not os.path.isfile(AFIR_LIT), reason="reference tree not present")
def test_reference_afir_lit_functions_translate():
    """The functions of the reference's AFIR round-trip test that use ops on this
    path (binary math, relu / neg / leaky_relu / abs, broadcast, sum, load /
    store, with their attribute dictionaries) translate one by one; an op
    outside the path is refused by name."""
    good = ["test_add", "test_sub", "test_mul", "test_div", "test_truediv", "test_minimum", "test_maximum",
            "test_relu", "test_neg", "test_leaky_relu", "test_abs", "test_abs_f16", "test_broadcast", "test_load",
            "test_store", "test_sum_reduce", "test_reduce_3d", "test_binary_1d", "test_binary_3d", "test_unary_1d",
            "test_unary_3d", "test_add_output_double_buffer", "test_abs_output_vector_out",
            "test_cast_f16_to_f32", "test_cast_f32_to_f16", "test_cast_output_vector_out"]
    for fn in good:
        p = subprocess.run([TR, "-mlir-to-hip", AFIR_LIT, "--function", fn], capture_output=True, text=True)
        assert p.returncode == 0, (fn, p.stderr)
        assert p.stdout.startswith(f"# kernel {fn}\nafir-hip-region 1\n") and p.stdout.rstrip().endswith("store\nend")
    for fn, op in (("test_exp", "afir.exp"), ("test_eq", "afir.eq")):
        p = subprocess.run([TR, "-mlir-to-hip", AFIR_LIT, "--function", fn], capture_output=True, text=True)
        assert p.returncode == 1 and f"{op} has no HIP lowering" in p.stderr, (fn, p.stderr)
    # a cast from an integer tensor is outside the float chains this backend lowers
    p = subprocess.run([TR, "-mlir-to-hip", AFIR_LIT, "--function", "test_cast"], capture_output=True, text=True)
    assert p.returncode == 1 and "integer and floating-point tensors" in p.stderr, p.stderr
    p = subprocess.run([TR, "-mlir-to-hip", AFIR_LIT, "--function", "nope"], capture_output=True, text=True)
    assert p.returncode == 1 and "no function @nope" in p.stderr


AFIR_CONVERSION = "/root/reference/test/Conversion/afir_to_ascir.mlir"


@pytest.mark.skipif(not os.path.isfile(AFIR_CONVERSION), reason="reference tree not present")
def test_reference_afir_conversion_functions_translate():
    """Every function of the reference's AFIR -> AscendC conversion test translates; its
    i32 addition and the round-trip test's i16 addition become integer regions."""
    import re
    names = re.findall(r"^func\.func @(\w+)", open(AFIR_CONVERSION).read(), re.M)
    assert "convert_add_i32" in names and len(names) >= 12
    for fn in names:
        p = subprocess.run([TR, "-mlir-to-hip", AFIR_CONVERSION, "--function", fn], capture_output=True, text=True)
        assert p.returncode == 0, (fn, p.stderr)
        assert p.stdout.startswith(f"# kernel {fn}\nafir-hip-region 1\n")
    def body(text):
        return [l.strip() for l in text.splitlines() if l.strip() and not l.startswith("#")]
    p = subprocess.run([TR, "-mlir-to-hip", AFIR_CONVERSION, "--function", "convert_add_i32"], capture_output=True, text=True)
    assert body(p.stdout) == body(RC.INT_ADD_I32)
    p = subprocess.run([TR, "-mlir-to-hip", AFIR_LIT, "--function", "test_add_i16"], capture_output=True, text=True)
    assert p.returncode == 0 and body(p.stdout) == body(RC.INT_ADD_I16)


def test_integer_afir_graph_matches_numpy():
    """relu(a - b) * a + (-b) on i32 tensors, against numpy's int32 arithmetic; ops that
    exist for floating point only are refused on integer tensors."""
    t = "tensor<?x?xi32>"
    rc, program, err = translate(MC.INT_CHAIN_I32)
    assert rc == 0, err
    rng = np.random.default_rng(3)
    a = rng.integers(-2**31, 2**31 - 1, (9, 21), dtype=np.int32)
    b = rng.integers(-2**31, 2**31 - 1, (9, 21), dtype=np.int32)
    with np.errstate(over="ignore"):
        want = np.maximum(a - b, np.int32(0)) * a + (-b)
    assert RO.evaluate(program, [a, b]).tobytes() == want.tobytes()
    for op, form in (("div", f"%a, %b : ({t}, {t}) -> {t}"), ("leaky_relu", f"%a {{negative_slop = 0.1 : f32}} : {t} -> {t}")):
        bad = f"func.func @f(%a : {t}, %b : {t}) -> {t} {{\n  %0 = afir.{op} {form}\n  return %0 : {t}\n}}\n"
        rc, _, err = translate(bad)
        assert rc == 1 and f"afir.{op} on integer tensors has no HIP lowering" in err, err
    mixed = ("func.func @f(%a : tensor<4xi32>, %b : tensor<4xf32>) -> tensor<4xf32> {\n"
             "  %0 = afir.add %a, %b : (tensor<4xi32>, tensor<4xf32>) -> tensor<4xf32>\n  return %0 : tensor<4xf32>\n}\n")
    rc, _, err = translate(mixed)
    assert rc == 1 and "integer and floating-point tensors in one operation" in err, err


def test_concat_of_three_parts_sums_the_row_offsets():
    out = program_of(MC.THREE_PART_CONCAT)
    offs = [l for l in out.splitlines() if l.startswith("outoff")]
    assert offs == ["outoff 0", "outoff arg0.0", "outoff arg0.0 arg1.0"]
    rng = np.random.default_rng(2)
    a, b, c = (rng.uniform(-1, 1, (r, 7)).astype(np.float32) for r in (3, 5, 2))
    want = np.concatenate([np.maximum(a, 0), -b, c], axis=0)
    assert RO.evaluate(out, [a, b, c]).tobytes() == want.tobytes()


def test_abs_is_maximum_of_x_and_minus_x():
    text = """func.func @a(%x: tensor<2x5xf32>) -> tensor<2x5xf32> {
  %0 = afir.abs %x : tensor<2x5xf32> -> tensor<2x5xf32>
  return %0 : tensor<2x5xf32>
}"""
    out = program_of(text)
    assert "push arg0 d0 d1\npush arg0 d0 d1\nneg\nmax\nstore" in out
    x = np.array([[-0.0, 0.0, -1.5, 2.0, -np.inf], [np.nan, 1e-40, -1e-40, 3.0, -3.0]], np.float32)
    got = RO.evaluate(out, [x])
    want = np.abs(x)
    assert ((got.view(np.uint32) == want.view(np.uint32)) | (np.isnan(got) & np.isnan(want))).all()


@pytest.mark.skipif(not os.path.isdir(REF_EXAMPLES), reason="reference tree not present")
def test_reference_matmul_example_translates():
    p = subprocess.run([TR, "-mlir-to-hip", os.path.join(REF_EXAMPLES, "matmul-add-leakyrelu", "step0_input.mlir")],
                       capture_output=True, text=True)
    assert p.returncode == 0, p.stderr
    assert "matmul arg0 arg1\npush arg2 d1\nadd\nleaky 0.00100000005\nstore" in p.stdout


def test_transposed_and_batched_matmul_ops(pkg):
    """linalg.matmul_transpose_a / _b and linalg.batch_matmul*: the other matmul-like ops of the
    reference's recogniser (AnnotateMixMatmulSemanticsPass.cpp:244-256) become 'matmul' with
    'ta' / 'tb', or open a rank-3 segment."""
    from ascend_mlir_amd import hip_kernels as H
    def body(mlir):
        return [l.strip() for l in program_of(mlir).splitlines() if l.strip() and not l.startswith("#")]
    b = body(MC.MATMUL_TRANSPOSE_A_F16)
    assert b[-3:] == ["matmul arg0 arg1 ta", "store", "end"] and "segment 2" in b
    b = body(MC.MATMUL_TRANSPOSE_B_F16)
    assert b[-3:] == ["matmul arg0 arg1 tb", "store", "end"]
    b = body(MC.MATMUL_TRANSPOSE_B_BIAS_LEAKY_BF16)
    assert b[-6:] == ["matmul arg0 arg1 tb", "push arg2 d1", "add", "leaky 0.0100097656", "store", "end"]   # 1e-2 as a bf16 constant
    b = body(MC.BATCH_MATMUL_BF16)
    assert b[-3:] == ["matmul arg0 arg1", "store", "end"] and "segment 3" in b
    assert [l for l in b if l.startswith("arg")] == ["arg in bf16 3", "arg in bf16 3", "arg in bf16 3", "arg out bf16 3"]
    b = body(MC.BATCH_MATMUL_TRANSPOSE_B_F16)
    assert b[-3:] == ["matmul arg0 arg1 tb", "store", "end"] and "segment 3" in b
    for mlir in (MC.MATMUL_TRANSPOSE_A_F16, MC.MATMUL_TRANSPOSE_B_BIAS_LEAKY_BF16, MC.BATCH_MATMUL_BF16,
                 MC.BATCH_MATMUL_TRANSPOSE_B_F16):
        r = H.Region(program_of(mlir))      # registers: the matmul kernels take it
        assert r.kernel.startswith("matmul_add_leakyrelu")
        r.close()
    # flags are part of the grammar: anything else after the operands is refused
    bad = program_of(MC.MATMUL_TRANSPOSE_B_F16).replace("matmul arg0 arg1 tb", "matmul arg0 arg1 tb ta")
    with pytest.raises(H.AfirHipError, match=r"\[ta\] \[tb\]"):
        H.Region(bad)


def _body(text):
    out = program_of(text)
    return [l.strip() for l in out.splitlines() if l.strip() and not l.startswith("#")]


def test_mixed_precision_chain_rounds_where_the_ir_truncates():
    """arith.truncf is a rounding to the narrower type ('cast f16'), arith.extf changes nothing;
    the last truncf to the output's own type is the store's rounding."""
    body = _body(MC.MIXED_PRECISION_CHAIN)
    assert body[body.index("outoff 0") + 1:] == [
        "push arg0 d0 d1", "cast f16", "push arg1 d1", "add", "push arg0 d0 d1", "mul", "store", "end"]
    rng = np.random.default_rng(8)
    a = rng.uniform(-3, 3, (5, 40)).astype(np.float32)
    b = rng.uniform(-3, 3, (40,)).astype(np.float16)
    want = ((a.astype(np.float16).astype(np.float32) + b.astype(np.float32)) * a).astype(np.float16)
    assert RO.evaluate(program_of(MC.MIXED_PRECISION_CHAIN), [a, b]).tobytes() == want.tobytes()
    # without the inner rounding the result differs: the cast is not decoration
    plain = ((a + b.astype(np.float32)) * a).astype(np.float16)
    assert plain.tobytes() != want.tobytes()


def test_named_linalg_ops_reshapes_and_float_casts():
    """linalg.transpose / add / broadcast / mul, a dense splat as init, expand_shape and
    collapse_shape of a unit dim, afir.cast down to bf16 and up again."""
    body = _body(MC.NAMED_OPS_GRAPH)
    assert body[body.index("outoff 0") + 1:] == [
        "push arg0 d0 d1", "push arg1 d1 d0", "add", "push arg2 d1", "mul", "cast bf16", "store", "end"]
    assert "size 4 8" in body
    rng = np.random.default_rng(9)
    a, b, c = (rng.uniform(-2, 2, s).astype(np.float32) for s in ((4, 8), (8, 4), (8,)))
    v = (a + b.T) * c[None, :]
    u = v.view(np.uint32)
    want = (((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16).astype(np.uint32).view(np.float32)     # bf16, nearest even
    assert RO.evaluate(program_of(MC.NAMED_OPS_GRAPH), [a, b, c]).tobytes() == want.tobytes()


def test_linalg_elementwise_with_broadcast_maps():
    body = _body(MC.ELEMENTWISE_KIND_SUB)
    assert body[body.index("outoff 0") + 1:] == ["push arg0 d1 d2", "push arg1 d0 0 d2", "sub", "store", "end"]
    assert "size arg2.0 arg2.1 arg2.2" in body
    for kind in ("tanh", "exp", "erf"):
        bad = subprocess.run([TR, "-mlir-to-hip", "-"], input=MC.ELEMENTWISE_KIND_SUB.replace("<sub>", f"<{kind}>"),
                             capture_output=True, text=True)
        assert bad.returncode == 1 and f"elementwise kind '{kind}' has no HIP lowering" in bad.stderr
    # reshapes that re-linearise, and dense constants that are not splats, are refused by name
    bad = subprocess.run([TR, "-mlir-to-hip", "-"], capture_output=True, text=True, input=MC.NAMED_OPS_GRAPH.replace(
        "[[0, 1], [2]] : tensor<4x1x8xf32> into tensor<4x8xf32>", "[[0, 1, 2]] : tensor<4x1x8xf32> into tensor<32xf32>"))
    assert bad.returncode == 1 and "merge or split dims of extent other than 1" in bad.stderr
    bad = subprocess.run([TR, "-mlir-to-hip", "-"], capture_output=True, text=True,
                         input=MC.NAMED_OPS_GRAPH.replace("dense<0.0> : tensor<4x8xf32>", "dense<[[1.0]]> : tensor<1x1xf32>"))
    assert bad.returncode == 1 and "other than splats" in bad.stderr


def test_named_reduce_and_unary_forms():
    """linalg.reduce with an addf combiner (region form and the short { arith.addf } form) is the
    row sum; linalg.square / reciprocal / copy are forms of mul / div / nothing."""
    body = _body(MC.NAMED_REDUCE_GRAPH)
    want_ops = ["const 1", "push arg0 d0 d1", "push arg0 d0 d1", "mul", "push arg1 d1", "add", "div", "reduce sum", "store", "end"]
    assert body[body.index("outoff 0") + 1:] == want_ops
    region_form = MC.NAMED_REDUCE_GRAPH
    a, b = region_form.index("  %red = linalg.reduce"), region_form.index("  return")
    short = (region_form[:a] + "  %red = linalg.reduce { arith.addf } ins(%cp : tensor<?x?xf32>) outs(%init : tensor<?xf32>) "
             "dimensions = [1]\n" + region_form[b:])
    assert _body(short) == body
    rng = np.random.default_rng(13)
    x, bias = rng.uniform(1, 2, (9, 300)).astype(np.float32), rng.uniform(0, 1, (300,)).astype(np.float32)
    got = RO.evaluate(program_of(MC.NAMED_REDUCE_GRAPH), [x, bias])
    ref = (1.0 / (x.astype(np.float64) ** 2 + bias.astype(np.float64))).sum(axis=1)
    assert got.dtype == np.float32 and np.allclose(got, ref, rtol=1e-5, atol=0)
    for frm, to, msg in (("arith.addf %in, %acc", "arith.mulf %in, %acc", "only a sum"),
                         ("dimensions = [1]", "dimensions = [0]", "innermost dim"),
                         ("arith.constant 0.0 : f32", "arith.constant 1.0 : f32", "zero-filled init")):
        bad = subprocess.run([TR, "-mlir-to-hip", "-"], input=region_form.replace(frm, to), capture_output=True, text=True)
        assert bad.returncode == 1 and msg in bad.stderr, (frm, bad.stderr)


LINALG_ADD_BROADCAST = "/root/reference/test/Dialect/AFIR/Transforms/linalgAddBroadcast.mlir"


@pytest.mark.skipif(not os.path.isfile(LINALG_ADD_BROADCAST), reason="reference tree not present")
def test_reference_linalg_add_broadcast_input_translates():
    """The input of the reference's --linalg-add-broadcast test (a linalg.elementwise add with
    broadcasting maps) translates as it stands; its tanh function is refused by kind."""
    p = subprocess.run([TR, "-mlir-to-hip", LINALG_ADD_BROADCAST, "--function", "unary_broadcast_addf"],
                       capture_output=True, text=True)
    assert p.returncode == 0, p.stderr
    body = [l.strip() for l in p.stdout.splitlines() if l.strip() and not l.startswith("#")]
    assert body[body.index("outoff 0") + 1:] == ["push arg0 d1 d2", "push arg1 d0 0 d2", "add", "store", "end"]
    rng = np.random.default_rng(10)
    a, c = rng.uniform(-1, 1, (16, 32)).astype(np.float32), rng.uniform(-1, 1, (8, 1, 32)).astype(np.float32)
    init = np.zeros((8, 16, 32), np.float32)
    assert RO.evaluate(p.stdout, [a, c, init]).tobytes() == (a[None] + c).tobytes()
    p = subprocess.run([TR, "-mlir-to-hip", LINALG_ADD_BROADCAST, "--function", "unary_broadcast_tanh"],
                       capture_output=True, text=True)
    assert p.returncode == 1 and "elementwise kind 'tanh' has no HIP lowering" in p.stderr
