"""The reference's example graphs end to end on the GPU, the way its
examples/*/run.sh drive them: kernel source (MLIR) -> runtime-session --kernel
-> artifact; seeded .npy inputs + golden -> run manifest -> runtime-session
--run-manifest --run; pass = the three session lines.  Shapes and tolerances
are the examples' own (run.sh atol / rtol lines); the MLIR is this repository's
text in the same syntax (tests/mlir_cases.py).  Needs a GPU."""
import json
import os
import subprocess

import numpy as np
import pytest

from oracle import afir_oracle as O
from tests import mlir_cases as MC
from tests import region_cases as RC

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
RS = os.path.join(ROOT, "ascend-mlir_amd", "bin", "runtime-session")
TR = os.path.join(ROOT, "ascend-mlir_amd", "bin", "afir-translate")


def _matmul_f16_case(m=128, k=256, n=128, seed=42):
    """Small integers: every product and partial sum is exact in float32, so
    the golden is independent of the summation order
    (examples/matmul-add-leakyrelu/gen_data.py:29-31)."""
    rng = np.random.default_rng(seed)
    a = rng.integers(-3, 4, (m, k)).astype(np.float16)
    b = rng.integers(-3, 4, (k, n)).astype(np.float16)
    bias = rng.integers(-8, 9, (n,)).astype(np.float32)
    init = np.zeros((m, n), np.float32)
    return None, [a, b, bias, init], O.matmul_bias_leakyrelu_f16(a, b, bias, 0.001)


def _int_chain_case(m=640, n=500, seed=42):
    """Full-range int32 values: every step wraps like numpy's int32 arrays."""
    rng = np.random.default_rng(seed)
    a = rng.integers(-2**31, 2**31 - 1, (m, n), dtype=np.int32)
    b = rng.integers(-2**31, 2**31 - 1, (m, n), dtype=np.int32)
    with np.errstate(over="ignore"):
        return None, [a, b], np.maximum(a - b, np.int32(0)) * a + (-b)


# (mlir, case, kernel kind, atol, rtol of the example's run.sh, bit-exact expected)
EXAMPLES = {
    "broadcast-add-reduce": (MC.ROW_BIAS_REDUCE, RC.case_reduce_rowbias, "vec", 10.0, 1e-2, False),
    "relu-broadcast-transpose": (MC.RELU_COLUMN_ADD, RC.case_relu_col_add, "vec", 1e-2, 1e-2, True),
    "gather-elementwise-fusion": (MC.RELU_GATHER_COLUMNS_ADD, RC.case_relu_colgather_add, "vec", 10.0, 1e-2, True),
    "matmul-add-leakyrelu": (MC.MATMUL_BIAS_LEAKY_F16, _matmul_f16_case, "mix", 1.0, 1e-2, True),
    "add-broadcast-concat": (MC.TWO_CHAINS_CONCAT, RC.case_add_broadcast_concat, "vec", 1e-3, 1e-3, True),
    "split-relu-brc-add-mul": (MC.SPLIT_HALVES, RC.case_split_relu_brc_add_mul, "vec", 1e-3, 1e-3, True),
    # not one of the reference's examples: its integer element types through the same pipeline
    "integer-chain": (MC.INT_CHAIN_I32, _int_chain_case, "vec", 0.0, 0.0, True),
}


def _rs(*args):
    return subprocess.run([RS, *args], capture_output=True, text=True, timeout=100)


@pytest.mark.parametrize("example", sorted(EXAMPLES))
def test_example_pipeline(tmp_path, example):
    mlir, case, kind, atol, rtol, exact = EXAMPLES[example]
    src = tmp_path / "step0_input.mlir"
    src.write_text(mlir)
    art = tmp_path / "artifact"
    p = _rs("--kernel", str(src), "--kernel-kind", kind, "--output", str(art), "--name", "kernel0")
    assert p.returncode == 0, p.stderr
    assert f"kernel_kind={kind}" in (art / "out" / "manifest.txt").read_text().splitlines()
    if kind != "mix":
        # the region was also emitted as HIP source and compiled for gfx950
        assert "code_object_path=kernel0.hsaco" in (art / "out" / "manifest.txt").read_text().splitlines()
        assert (art / "kernel0.hip").stat().st_size > 0 and (art / "kernel0.hsaco").stat().st_size > 0
    ts = tmp_path / "tiling_space.json"
    assert subprocess.run([TR, "-mlir-to-hip", str(src), "-o", str(tmp_path / "program.txt"),
                           "--tiling-space-out", str(ts)]).returncode == 0
    _, inputs, want = case()
    want = np.ascontiguousarray(want)     # fancy indexing may hand back Fortran order
    bind = []
    for i, x in enumerate(inputs):
        np.save(tmp_path / f"input_{i}.npy", x)
        bind.append({"name": f"in{i}", "path": str(tmp_path / f"input_{i}.npy")})
    np.save(tmp_path / "output_expected.npy", want)
    fields = [f["name"] for f in json.loads(ts.read_text())["tiling_params"]]
    dims = [d for x in inputs for d in x.shape] + list(want.shape)
    assert len(fields) == len(dims)
    manifest = {
        "task_id": "main", "backend": "hip", "artifact_root": str(art), "inputs": bind,
        "outputs": [{"name": "out", "path": str(tmp_path / "output_actual.npy")}],
        "expected_outputs": [{"name": "out", "path": str(tmp_path / "output_expected.npy")}],
        "tiling": {"schema": str(ts), "params": ",".join(f"{k}={v}" for k, v in zip(fields, dims))},
        "block_dim": 0, "workspace_size": 8192, "profiling": False, "atol": atol, "rtol": rtol}
    (tmp_path / "run_manifest.json").write_text(json.dumps(manifest))
    p = _rs("--run-manifest", str(tmp_path / "run_manifest.json"), "--run")
    assert p.returncode == 0, p.stdout + p.stderr
    lines = p.stdout.splitlines()
    for line in ("session.backend=hip", "session.result=success", "session.validation=pass"):
        assert line in lines, p.stdout
    got = np.load(tmp_path / "output_actual.npy")
    if exact:
        assert got.tobytes() == want.tobytes()
    else:   # float32 row sums in another order, rounded to f16: within one f16 ulp
        assert np.all(np.abs(got.astype(np.float64) - want.astype(np.float64))
                      <= 2.0 ** -10 * np.abs(want.astype(np.float64)) + 1e-3)
    if kind != "mix":
        # the same artifact on the interpreter kernel instead of its code object
        manifest["outputs"][0]["path"] = str(tmp_path / "output_interpreted.npy")
        (tmp_path / "run_manifest2.json").write_text(json.dumps(manifest))
        p = subprocess.run([RS, "--run-manifest", str(tmp_path / "run_manifest2.json"), "--run"],
                           capture_output=True, text=True, timeout=100,
                           env=dict(os.environ, AFIR_HIP_REGION_INTERPRET="1"))
        assert p.returncode == 0, p.stdout + p.stderr
        other = np.load(tmp_path / "output_interpreted.npy")
        if exact:
            assert other.tobytes() == got.tobytes()
        else:
            assert np.all(np.abs(other.astype(np.float64) - got.astype(np.float64))
                          <= 2.0 ** -9 * np.abs(want.astype(np.float64)) + 2e-3)


def test_capi_runs_a_compiled_mlir_kernel(pkg, tmp_path):
    """compile_kernel on MLIR text, then execute_kernel on host arrays: the
    reference's python/test/test_runtime_e2e.py flow."""
    from ascend_mlir_amd import runtime as R
    src = tmp_path / "k.mlir"
    src.write_text(MC.SPLIT_HALVES)
    path = R.compile_kernel(src, tmp_path / "art", "split_halves")
    _, inputs, want = RC.case_split_relu_brc_add_mul(64, 40)
    dims = [d for x in inputs for d in x.shape] + list(want.shape)
    import struct
    tiling = struct.pack("<%dq" % len(dims), *dims)
    ex = R.KernelExecutor(device_id=0)
    out = ex.execute(R.read_binary(path), "split_halves", inputs, [np.empty_like(want)], tiling)
    assert out[0].tobytes() == want.tobytes()
    with pytest.raises(R.ExecutorError, match="tiling data implies"):
        ex.execute(R.read_binary(path), "split_halves", inputs, [np.empty((10, 40), np.float16)], tiling)


def test_fast_paths_and_generic_kernel_agree(pkg, monkeypatch):
    """A program that is one of the hand-tuned kernels gives the same bits on
    that kernel and on the generic one (row sums: same tolerance both ways)."""
    import torch
    from ascend_mlir_amd import hip_kernels as H
    H.load()
    for name, case in [("c1", RC.case_c1), ("c3", RC.case_c3), ("c4", RC.case_c4), ("c2", RC.case_c2)]:
        text, inputs, want = case()
        outs = {}
        for generic in ("0", "1"):
            monkeypatch.setenv("AFIR_HIP_REGION_GENERIC", generic)
            r = H.Region(text)
            assert (r.kernel == "fused_region") == (generic == "1")
            dev = [torch.from_numpy(x).cuda() for x in inputs]
            outs[generic] = r(*dev, out_shape=want.shape).cpu().numpy()
            r.close()
        if name == "c2":
            assert np.allclose(outs["0"], outs["1"], rtol=1e-5, atol=1e-3)
        else:
            assert outs["0"].tobytes() == outs["1"].tobytes() == want.tobytes()


def test_matmul_bf16_program_runs_on_the_mfma_kernel(pkg):
    import torch
    from ascend_mlir_amd import hip_kernels as H
    H.load()
    p = subprocess.run([TR, "-mlir-to-hip", "-"], input=MC.MATMUL_BIAS_LEAKY_BF16, capture_output=True, text=True)
    assert p.returncode == 0, p.stderr
    r = H.Region(p.stdout)
    assert r.kernel == "matmul_add_leakyrelu"
    a, b, bias = O.gen_c5(256, 512, 256)

    def dev(bits):
        return torch.from_numpy(bits.view(np.int16)).cuda().view(torch.bfloat16)
    init = torch.zeros((256, 256), dtype=torch.bfloat16, device="cuda")
    out = r(dev(a), dev(b), dev(bias), init, out_shape=(256, 256))
    got = out.view(torch.int16).cpu().numpy().view(np.uint16)
    res = O.compare_outputs([(got, "bf16")], [(O.golden_c5(a, b, bias, 0.01), "bf16")], 1e-5, 1e-2)
    assert res["passed"], res
    assert O.nonfinite_mismatches(got, O.golden_c5(a, b, bias, 0.01), "bf16") == 0
    r.close()


def test_two_kernel_session_feeds_one_kernel_into_the_next(tmp_path):
    """A two-task manifest (the shape of examples/real-npu-multikernel): t = (a + b) * b on the first
    kernel, y[i] = sum_j (t[i,j] + bias[j]) on the second, the intermediate tensor bound as a task output."""
    k1, k2 = tmp_path / "k1.mlir", tmp_path / "k2.mlir"
    k1.write_text(MC.C1_AFIR)
    k2.write_text(MC.C2_LINALG)
    for src, name in ((k1, "add_mul"), (k2, "rowsum")):
        assert _rs("--kernel", str(src), "--output", str(tmp_path / name), "--name", name).returncode == 0
        assert subprocess.run([TR, "-mlir-to-hip", str(src), "-o", str(tmp_path / (name + ".txt")),
                               "--tiling-space-out", str(tmp_path / (name + ".json"))]).returncode == 0
    rng = np.random.default_rng(3)
    m, n = 300, 1000
    a = rng.uniform(-1, 1, (m, n)).astype(np.float32)
    b = rng.uniform(-1, 1, (m, n)).astype(np.float32)
    bias = rng.uniform(-1, 1, (n,)).astype(np.float32)
    t = (a + b) * b
    want = (t + bias[None, :]).sum(axis=1, dtype=np.float32)
    for name, arr in (("a", a), ("b", b), ("bias", bias), ("want", want)):
        np.save(tmp_path / f"{name}.npy", arr)

    def params(path, dims):
        fields = [f["name"] for f in json.loads(open(path).read())["tiling_params"]]
        return ",".join(f"{k}={v}" for k, v in zip(fields, dims))
    manifest = {"backend": "hip", "tasks": [
        {"task_id": "reduce", "artifact_root": str(tmp_path / "rowsum"), "dependencies": ["chain"],
         "inputs": [{"name": "x", "source": "task_output", "upstream_task": "chain", "upstream_output": "t"},
                    {"name": "bias", "path": str(tmp_path / "bias.npy")}],
         "outputs": [{"name": "y", "path": str(tmp_path / "y.npy")}],
         "expected_outputs": [{"name": "y", "path": str(tmp_path / "want.npy")}],
         "tiling": {"schema": str(tmp_path / "rowsum.json"), "params": params(tmp_path / "rowsum.json", [m, n, n, m])},
         "atol": 1e-3, "rtol": 1e-5, "profiling": True},
        {"task_id": "chain", "artifact_root": str(tmp_path / "add_mul"), "profiling": True,
         "inputs": [{"name": "a", "path": str(tmp_path / "a.npy")}, {"name": "b", "path": str(tmp_path / "b.npy")}],
         "outputs": [{"name": "t", "shape": [m, n], "dtype": "f32"}],
         "tiling": {"schema": str(tmp_path / "add_mul.json"),
                    "params": params(tmp_path / "add_mul.json", [m, n, m, n, m, n])}}]}
    (tmp_path / "m.json").write_text(json.dumps(manifest))
    (tmp_path / "tmp").mkdir()
    p = subprocess.run([RS, "--run-manifest", str(tmp_path / "m.json"), "--run"], capture_output=True, text=True,
                       timeout=100, env=dict(os.environ, TMPDIR=str(tmp_path / "tmp")))
    assert p.returncode == 0, p.stdout + p.stderr
    lines = p.stdout.splitlines()
    assert "session.plan[0]=chain" in lines and "session.plan[1]=reduce" in lines
    # both tasks profiled: measured kernel times in the traces and the retained summary
    kv = dict(l.split("=", 1) for l in lines if "=" in l)
    assert kv["session.profile.count"] == "2"
    traces = [json.loads(open(kv[f"session.profile[{i}]"]).read()) for i in range(2)]
    assert [t_["task_id"] for t_ in traces] == ["chain", "reduce"]
    assert all(t_["backend"] == "hip" and 0 < t_["score"] < 10_000_000 and t_["validation_passed"] for t_ in traces)
    summary = json.loads(open(kv["session.profile.summary"]).read())
    assert summary["task_count"] == 2 and summary["total_score"] == sum(t_["score"] for t_ in traces)
    assert "session.result=success" in lines and "session.validation=pass" in lines
    assert np.load(tmp_path / "chain__t.npy").tobytes() == t.tobytes()      # the intermediate is bit-exact
    assert np.allclose(np.load(tmp_path / "y.npy"), want, rtol=1e-5, atol=1e-3)


@pytest.mark.parametrize("kind", ["none", "bias", "bias_relu", "relu"])
@pytest.mark.parametrize("ty", ["f16", "bf16"])
def test_matmul_epilogue_kinds(pkg, kind, ty):
    """matmul with no epilogue, with a bias add only (the reference's epilogue
    kinds "None" and "BiasAdd"), with bias add and relu (its runtime's
    "BiasAddRelu") and with relu alone, on the MFMA kernels.  Small-integer operands:
    every product and partial sum is exact in float32
    (examples/matmul-add-leakyrelu/gen_data.py:29-31), so the result does not
    depend on the order of accumulation; negative sums keep their sign without a
    leaky relu.  2048x256x4096 (128 tiles of 256x256) takes the direct-to-LDS kernel,
    512x256x512 the register-staged one with 128x128 tiles, 96x64x40 its bounds-checked form."""
    import torch
    from ascend_mlir_amd import hip_kernels as H
    from oracle import region_oracle as RO
    H.load()
    mlir = {("none", "f16"): MC.MATMUL_PLAIN_F16, ("bias", "f16"): MC.MATMUL_BIAS_F16,
            ("none", "bf16"): MC.MATMUL_PLAIN_BF16, ("bias", "bf16"): MC.MATMUL_BIAS_BF16,
            ("bias_relu", "f16"): MC.MATMUL_BIAS_RELU_F16, ("bias_relu", "bf16"): MC.MATMUL_BIAS_RELU_BF16,
            ("relu", "f16"): MC.MATMUL_RELU_F16, ("relu", "bf16"): MC.MATMUL_RELU_BF16}[(kind, ty)]
    has_bias = kind in ("bias", "bias_relu")
    p = subprocess.run([TR, "-mlir-to-hip", "-"], input=mlir, capture_output=True, text=True)
    assert p.returncode == 0, p.stderr
    for (m, k, n) in ((512, 256, 512), (96, 64, 40), (2048, 256, 4096)):
        rng = np.random.default_rng(7)
        a = rng.integers(-3, 4, (m, k)).astype(np.float32)
        b = rng.integers(-3, 4, (k, n)).astype(np.float32)
        bias = rng.integers(-8, 9, (n,)).astype(np.float32)
        exact = a @ b + (bias[None, :] if has_bias else 0.0)      # integers: exact in float32
        if kind.endswith("relu"):
            exact = np.maximum(exact, 0.0) + 0.0          # +0 where the sum is negative or zero
        assert np.abs(exact).max() < 2 ** 24
        if ty == "f16":
            ins = [a.astype(np.float16), b.astype(np.float16)] + ([bias] if has_bias else [])
            init = np.zeros((m, n), np.float32)
            want = exact.astype(np.float32)
            dev = [torch.from_numpy(x).cuda() for x in ins + [init]]
        else:
            ins = [O.f32_to_bf16_bits(a), O.f32_to_bf16_bits(b)] + ([O.f32_to_bf16_bits(bias)] if has_bias else [])
            init = O.f32_to_bf16_bits(np.zeros((m, n), np.float32))
            want = O.f32_to_bf16_bits(exact.astype(np.float32))
            dev = [torch.from_numpy(x.view(np.int16)).cuda().view(torch.bfloat16) for x in ins + [init]]
        assert RO.evaluate(p.stdout, ins + [init]).tobytes() == want.tobytes()      # the oracle agrees with the closed form
        r = H.Region(p.stdout)
        out = r(*dev, out_shape=(m, n))
        got = out.cpu().numpy() if ty == "f16" else out.view(torch.int16).cpu().numpy().view(np.uint16)
        r.close()
        assert got.tobytes() == want.tobytes(), (kind, ty, m, k, n)


def _multikernel_artifacts(tmp_path):
    for name, text in (("const640", RC.CONST_ONE), ("const_with_input640", RC.CONST_TWO_IGNORING_INPUT),
                       ("copy_scalar640", RC.COPY_1D), ("add_wait640", RC.ADD_1D)):
        src = tmp_path / f"{name}.region"
        src.write_text(text)
        p = _rs("--kernel", str(src), "--output", str(tmp_path / "artifacts" / name / "artifact"), "--name", name)
        assert p.returncode == 0, p.stderr
    return tmp_path / "artifacts"


@pytest.mark.parametrize("case", ["serial-two-kernel", "fork-join"])
def test_reference_multikernel_manifests(tmp_path, case):
    """The two task graphs of examples/real-npu-multikernel (prepare.sh:74-176) with their own
    shapes, bindings and goldens (gen_data.py:17-33: 640 x 1.0 after const -> copy, 640 x 3.0
    after const(1) + const(2)); the kernels are hand-written there and region programs here.
    No task has a tiling binding: extents come from the bound tensors."""
    arts = _multikernel_artifacts(tmp_path)
    common = {"block_dim": 1, "workspace_size": 16384, "atol": 0, "rtol": 0}
    out = tmp_path / case
    out.mkdir()
    if case == "serial-two-kernel":
        np.save(out / "expected.npy", np.full((640,), 1.0, np.float16))
        tasks = [
            dict(task_id="producer", artifact_root=str(arts / "const640" / "artifact"),
                 outputs=[{"name": "mid", "shape": [640], "dtype": "f16"}], **common),
            dict(task_id="consumer", artifact_root=str(arts / "copy_scalar640" / "artifact"), dependencies=["producer"],
                 inputs=[{"name": "input", "source": "task_output", "upstream_task": "producer", "upstream_output": "mid"}],
                 outputs=[{"name": "out", "path": str(out / "output.npy"), "shape": [640], "dtype": "f16"}],
                 expected_outputs=[{"name": "out", "path": str(out / "expected.npy")}], **common)]
        plan = ["producer", "consumer"]
    else:
        np.save(out / "expected.npy", np.full((640,), 3.0, np.float16))
        np.save(out / "input.npy", (np.arange(640) / 17.0).astype(np.float16))
        tasks = [
            dict(task_id="producer_a", artifact_root=str(arts / "const640" / "artifact"),
                 outputs=[{"name": "a", "shape": [640], "dtype": "f16"}], **common),
            dict(task_id="producer_b", artifact_root=str(arts / "const_with_input640" / "artifact"),
                 inputs=[{"name": "input", "path": str(out / "input.npy")}],
                 outputs=[{"name": "b", "shape": [640], "dtype": "f16"}], **common),
            dict(task_id="consumer", artifact_root=str(arts / "add_wait640" / "artifact"),
                 dependencies=["producer_a", "producer_b"],
                 inputs=[{"name": "lhs", "source": "task_output", "upstream_task": "producer_a", "upstream_output": "a"},
                         {"name": "rhs", "source": "task_output", "upstream_task": "producer_b", "upstream_output": "b"}],
                 outputs=[{"name": "out", "path": str(out / "output.npy"), "shape": [640], "dtype": "f16"}],
                 expected_outputs=[{"name": "out", "path": str(out / "expected.npy")}], **common)]
        plan = ["producer_a", "producer_b", "consumer"]
    (out / "run_manifest.json").write_text(json.dumps({"backend": "hip", "tasks": tasks}))
    p = _rs("--run-manifest", str(out / "run_manifest.json"), "--run")
    assert p.returncode == 0, p.stdout + p.stderr
    lines = p.stdout.splitlines()
    assert [l.split("=")[1] for l in lines if l.startswith("session.plan[")] == plan
    for line in ("session.backend=hip", "session.result=success", "session.validation=pass"):
        assert line in lines, p.stdout
    assert np.load(out / "output.npy").tobytes() == np.load(out / "expected.npy").tobytes()


def test_asc_graph_form_runs_interpreted_and_compiled(pkg, monkeypatch, tmp_path):
    """The AscGraph form (load / broadcast / add / mul / sub / store) through the
    translator onto the GPU, on the interpreter kernel and on its compiled kernel."""
    import torch
    from ascend_mlir_amd import hip_kernels as H
    from oracle import region_oracle as RO
    H.load()
    p = subprocess.run([TR, "-mlir-to-hip", "-"], input=MC.ASC_GRAPH_FORM, capture_output=True, text=True)
    assert p.returncode == 0, p.stderr
    rng = np.random.default_rng(4)
    x = rng.uniform(-2, 2, (12, 40)).astype(np.float32)
    y = rng.uniform(-2, 2, (1, 40)).astype(np.float32)
    want = RO.evaluate(p.stdout, [x, y])
    r = H.Region(p.stdout)
    dev = [torch.from_numpy(x).cuda(), torch.from_numpy(y).cuda()]
    assert r(*dev, out_shape=(12, 40)).cpu().numpy().tobytes() == want.tobytes()
    r.compile(cache_dir=str(tmp_path))
    assert r.kernel == "fused_region_compiled"
    assert r(*dev, out_shape=(12, 40)).cpu().numpy().tobytes() == want.tobytes()
    r.close()


def test_concat_of_three_parts_runs_interpreted_and_compiled(pkg, tmp_path):
    import torch
    from ascend_mlir_amd import hip_kernels as H
    H.load()
    p = subprocess.run([TR, "-mlir-to-hip", "-"], input=MC.THREE_PART_CONCAT, capture_output=True, text=True)
    assert p.returncode == 0, p.stderr
    rng = np.random.default_rng(2)
    a, b, c = (rng.uniform(-1, 1, (r, 70)).astype(np.float32) for r in (33, 5, 120))
    want = np.concatenate([np.maximum(a, 0), -b, c], axis=0)
    r = H.Region(p.stdout)
    dev = [torch.from_numpy(x).cuda() for x in (a, b, c)]
    assert r(*dev, out_shape=want.shape).cpu().numpy().tobytes() == want.tobytes()
    r.compile(cache_dir=str(tmp_path))        # three segments in one launch
    assert "afir_region_all_i32_g" in r.emit_source()
    assert r(*dev, out_shape=want.shape).cpu().numpy().tobytes() == want.tobytes()
    r.close()
