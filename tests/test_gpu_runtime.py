"""The fused kernels reached the way the reference's callers reach a kernel:
through afirt_compiler_* / afirt_executor_* with host buffers and packed tiling
bytes (reference callers: python/runtime/executor.py:177-241,
test/tools/runtime/test_capi_runtime.cpp:93-199) and through
`runtime-session --run-manifest M --run` on .npy files
(examples/broadcast-add-reduce/run.sh:226-273).  Needs a GPU."""
import json
import os
import subprocess

import numpy as np
import pytest

from oracle import afir_oracle as O

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
RS = os.path.join(ROOT, "ascend-mlir_amd", "bin", "runtime-session")


@pytest.fixture(scope="module")
def R(pkg):
    from ascend_mlir_amd import runtime
    return runtime


@pytest.fixture(scope="module")
def executor(R):
    ex = R.KernelExecutor(device_id=0)
    ex.initialize()
    return ex


def _descriptor(tmp_path, family):
    src = tmp_path / f"{family}.txt"
    src.write_text(f"hip_kernel={family}\n")
    return src


def _compile(R, tmp_path, family, name=None):
    path = R.compile_kernel(_descriptor(tmp_path, family), tmp_path / f"art_{family}", name or family)
    return path, R.read_binary(path)


def _cases():
    a, b = O.gen_c1((300, 1000))
    yield ("fused_add_mul", [a, b], [np.empty_like(a)], dict(dim_arg0_0=300, dim_arg0_1=1000),
           [O.golden_c1(a, b)], "f32", 0.0, 0.0)
    x, bias = O.gen_c2(96, 4096)
    want = O.golden_c2(x, bias)
    yield ("broadcast_add_reducesum", [x, bias], [np.empty(96, np.float32)],
           dict(dim_arg0_0=96, dim_arg0_1=4096), [want], "f32", 1e-3, 1e-5)
    x, c = O.gen_c3(3, 256, 128)
    yield ("relu_broadcast_add_transpose", [x, c], [np.empty((3, 128, 256), np.float16)],
           dict(dim_arg0_0=3, dim_arg0_1=256, dim_arg0_2=128), [O.golden_c3(x, c)], "f16", 0.0, 0.0)
    table, idx, scale, shift = O.gen_c4(4096, 1024, 1000)
    yield ("gather_scale_shift", [table, idx, scale, shift], [np.empty((1000, 1024), np.float16)],
           dict(dim_arg0_0=4096, dim_arg0_1=1024, dim_arg1_0=1000),
           [O.golden_c4(table, idx, scale, shift)], "f16", 0.0, 0.0)
    am, bm, biasm = O.gen_c5(512, 512, 256)
    alpha_bits = int(np.float32(0.01).view(np.uint32))
    yield ("matmul_add_leakyrelu", [am, bm, biasm], [np.empty((512, 256), np.uint16)],
           dict(dim_arg0_0=512, dim_arg0_1=512, dim_arg1_1=256, alpha_f32_bits=alpha_bits),
           [O.golden_c5(am, bm, biasm, 0.01)], "bf16", 1e-5, 1e-2)


CASES = list(_cases())


@pytest.mark.parametrize("case", CASES, ids=[c[0] for c in CASES])
def test_capi_run_matches_oracle(R, executor, tmp_path, case):
    family, inputs, outputs, dims, want, dt, atol, rtol = case
    path, binary = _compile(R, tmp_path, family)
    tiling = R.TilingSchema.for_kernel(family).pack(**dims)
    got = executor.execute(binary, family, inputs, outputs, tiling)
    r = O.compare_outputs([(got[0], dt)], [(want[0], dt)], atol, rtol)
    assert r["passed"], r
    if atol == 0.0 and rtol == 0.0:
        assert got[0].tobytes() == want[0].tobytes()


def test_capi_run_file_and_cube_magic(R, executor, tmp_path):
    """afirt_executor_run_file reads the artifact itself; both magics are
    accepted and anything else is refused (lib/CAPI/Runtime/Runtime.cpp:113-120)."""
    import ctypes
    L = R.load_capi()
    path, _ = _compile(R, tmp_path, "fused_add_mul", "my_kernel")
    a, b = O.gen_c1((17, 33))
    out = np.zeros_like(a)
    tiling = R.TilingSchema.for_kernel("fused_add_mul").pack(dim_arg0_0=17, dim_arg0_1=33)
    vp, sz = ctypes.c_void_p, ctypes.c_size_t
    inp = (vp * 2)(a.ctypes.data, b.ctypes.data)
    inb = (sz * 2)(a.nbytes, b.nbytes)
    outp, outb = (vp * 1)(out.ctypes.data), (sz * 1)(out.nbytes)
    til = (ctypes.c_uint8 * len(tiling)).from_buffer_copy(tiling)
    err = ctypes.create_string_buffer(512)
    for magic in (R.MAGIC_ELF_AIVEC, R.MAGIC_ELF_AICUBE):
        out[...] = 0
        rc = L.afirt_executor_run_file(executor.runtime._handle, str(path).encode(), b"my_kernel", 2,
                                       inp, inb, 1, outp, outb, til, len(tiling), 0, magic, err,
                                       len(err))
        assert rc == 0, err.value
        assert out.tobytes() == O.golden_c1(a, b).tobytes()
    rc = L.afirt_executor_run_file(executor.runtime._handle, str(path).encode(), b"my_kernel", 2,
                                   inp, inb, 1, outp, outb, til, len(tiling), 0, 0x12345678, err,
                                   len(err))
    assert rc != 0 and b"magic" in err.value


def test_capi_rejects_buffers_that_do_not_match_the_tiling(R, executor, tmp_path):
    _, binary = _compile(R, tmp_path, "fused_add_mul")
    a, b = O.gen_c1((8, 8))
    sch = R.TilingSchema.for_kernel("fused_add_mul")
    with pytest.raises(R.ExecutorError, match="tiling data implies"):
        executor.execute(binary, "fused_add_mul", [a, b], [np.empty((8, 8), np.float32)],
                         sch.pack(dim_arg0_0=8, dim_arg0_1=16))
    with pytest.raises(R.ExecutorError, match="expects 2 inputs"):
        executor.execute(binary, "fused_add_mul", [a], [np.empty((8, 8), np.float32)],
                         sch.pack(dim_arg0_0=8, dim_arg0_1=8))
    with pytest.raises(R.ExecutorError, match="tiling"):
        executor.execute(binary, "fused_add_mul", [a, b], [np.empty((8, 8), np.float32)], b"\x01\x02")
    with pytest.raises(R.ExecutorError, match="artifact"):
        executor.execute(b"not an artifact", "fused_add_mul", [a, b],
                         [np.empty((8, 8), np.float32)], sch.pack(dim_arg0_0=8, dim_arg0_1=8))
    # the executor is still usable after refused calls
    got = executor.execute(binary, "fused_add_mul", [a, b], [np.empty((8, 8), np.float32)],
                           sch.pack(dim_arg0_0=8, dim_arg0_1=8))
    assert got[0].tobytes() == O.golden_c1(a, b).tobytes()


def test_capi_gather_index_out_of_range_is_an_error(R, executor, tmp_path):
    _, binary = _compile(R, tmp_path, "gather_scale_shift")
    table, idx, scale, shift = O.gen_c4(128, 64, 40)
    idx = idx.copy()
    idx[7] = 128
    tiling = R.TilingSchema.for_kernel("gather_scale_shift").pack(dim_arg0_0=128, dim_arg0_1=64,
                                                                  dim_arg1_0=40)
    with pytest.raises(R.ExecutorError, match="index out of range"):
        executor.execute(binary, "gather_scale_shift", [table, idx, scale, shift],
                         [np.empty((40, 64), np.float16)], tiling)


# ------------------------------------------------------- runtime-session CLI --

def _rs(*args):
    return subprocess.run([RS, *args], capture_output=True, text=True, timeout=100)


def _save(path, arr, dt):
    if dt == "bf16":
        O.save_npy(str(path), arr, "bf16")
    else:
        np.save(path, arr)


@pytest.mark.parametrize("case", CASES, ids=[c[0] for c in CASES])
def test_cli_run_manifest_validates_on_gpu(tmp_path, case):
    family, inputs, outputs, dims, want, dt, atol, rtol = case
    src = _descriptor(tmp_path, family)
    kind = "mix" if family == "matmul_add_leakyrelu" else "vec"
    art = tmp_path / "artifact"
    p = _rs("--kernel", str(src), "--kernel-kind", kind, "--output", str(art), "--name", family)
    assert p.returncode == 0, p.stderr
    in_dt = "bf16" if dt == "bf16" else None
    bind = []
    for i, x in enumerate(inputs):
        f = tmp_path / f"input_{i}.npy"
        _save(f, x, in_dt)
        bind.append({"name": f"in{i}", "path": str(f)})
    _save(tmp_path / "expected.npy", want[0], in_dt)
    fields = [{"name": k} for k in dims]
    (tmp_path / "tiling_space.json").write_text(json.dumps({"tiling_params": fields}))
    manifest = {
        "task_id": "main", "backend": "hip", "artifact_root": str(art), "inputs": bind,
        "outputs": [{"name": "out", "path": str(tmp_path / "output_actual.npy")}],
        "expected_outputs": [{"name": "out", "path": str(tmp_path / "expected.npy")}],
        "tiling": {"schema": str(tmp_path / "tiling_space.json"),
                   "params": ",".join(f"{k}={v}" for k, v in dims.items())},
        "block_dim": 0, "profiling": True, "atol": atol, "rtol": rtol}
    (tmp_path / "run_manifest.json").write_text(json.dumps(manifest))
    p = _rs("--run-manifest", str(tmp_path / "run_manifest.json"), "--run")
    assert p.returncode == 0, p.stdout + p.stderr
    lines = p.stdout.splitlines()
    for line in ("session.backend=hip", "session.result=success", "session.validation=pass"):
        assert line in lines, p.stdout
    if dt == "bf16":
        got, gdt = O.load_npy(str(tmp_path / "output_actual.npy"))
        assert gdt == "bf16"
    else:
        got = np.load(tmp_path / "output_actual.npy")
    r = O.compare_outputs([(got.reshape(want[0].shape), dt)], [(want[0], dt)], atol, rtol)
    assert r["passed"], r


def test_cli_validation_failure_exit_code(tmp_path):
    src = _descriptor(tmp_path, "fused_add_mul")
    art = tmp_path / "artifact"
    assert _rs("--kernel", str(src), "--output", str(art), "--name", "k").returncode == 0
    a, b = O.gen_c1((4, 4))
    np.save(tmp_path / "a.npy", a)
    np.save(tmp_path / "b.npy", b)
    np.save(tmp_path / "e.npy", O.golden_c1(a, b) + np.float32(1.0))
    (tmp_path / "ts.json").write_text(json.dumps(
        {"tiling_params": [{"name": "dim_arg0_0"}, {"name": "dim_arg0_1"}]}))
    m = {"task_id": "main", "backend": "hip", "artifact_root": str(art),
         "inputs": [{"name": "a", "path": str(tmp_path / "a.npy")},
                    {"name": "b", "path": str(tmp_path / "b.npy")}],
         "outputs": [{"name": "o", "path": str(tmp_path / "o.npy")}],
         "expected_outputs": [{"name": "o", "path": str(tmp_path / "e.npy")}],
         "tiling": {"schema": str(tmp_path / "ts.json"), "params": "dim_arg0_0=4,dim_arg0_1=4"},
         "atol": 1e-6, "rtol": 0}
    (tmp_path / "m.json").write_text(json.dumps(m))
    p = _rs("--run-manifest", str(tmp_path / "m.json"), "--run")
    assert p.returncode == 2
    assert "session.validation=fail" in p.stderr and "session.error_stage=validate" in p.stderr


# ------------------------------------- block_dim of the reference's callers --

def _full_size(family):
    if family == "fused_add_mul":
        a, b = O.gen_c1((4096, 4096))
        return ([a, b], np.empty_like(a), dict(dim_arg0_0=4096, dim_arg0_1=4096), O.golden_c1(a, b))
    table, idx, scale, shift = O.gen_c4(131072, 1024, 32768)
    return ([table, idx, scale, shift], np.empty((32768, 1024), np.float16),
            dict(dim_arg0_0=131072, dim_arg0_1=1024, dim_arg1_0=32768), O.golden_c4(table, idx, scale, shift))


@pytest.mark.parametrize("family", ["fused_add_mul", "gather_scale_shift"])
def test_reference_block_dim_values_do_not_size_the_grid(R, executor, tmp_path, family):
    """The reference's callers pass an Ascend AI-core count as block_dim: 1 by default
    (python/runtime/executor.py:183), 8 (test/tools/runtime/test_capi_runtime.cpp:171-174),
    40 (examples/broadcast-add-reduce/run.sh:259).  Through afirt_executor_run those values must
    reach the same kernel on the same grid, at the same speed, as the launcher's own choice, at
    the benchmark's full size, bit-exact against the oracle."""
    _, binary = _compile(R, tmp_path, family)
    inputs, out, dims, want = _full_size(family)
    tiling = R.TilingSchema.for_kernel(family).pack(**dims)
    seen = {}
    # the fastest of several per value, the values taking turns: a launch that follows a host copy
    # runs at whatever clocks the device has reached, and drifts of that kind hit every value alike;
    # at least three turns, and more (up to twelve) while a value has not yet had a launch as fast
    # as the launcher's own choice
    for turn in range(12):
        if turn >= 3 and all(seen[v]["kernel_ns"] <= 1.10 * seen[0]["kernel_ns"] for v in (1, 8, 40)):
            break
        for block_dim in (0, 1, 8, 40):
            out[...] = 0
            got = executor.execute(binary, family, inputs, [out], tiling, block_dim=block_dim)
            assert got[0].tobytes() == want.tobytes(), block_dim
            note = executor.runtime.last_launch()
            best = seen.get(block_dim)
            seen[block_dim] = note if best is None or note["kernel_ns"] < best["kernel_ns"] else best
    base = seen[0]
    assert base["workgroups"] >= 1024 and "phased" in base["kernel"], base
    for block_dim in (1, 8, 40):
        s = seen[block_dim]
        assert (s["kernel"], s["workgroups"], s["threads"]) == (base["kernel"], base["workgroups"], base["threads"])
        assert s["kernel_ns"] <= 1.10 * base["kernel_ns"], (block_dim, s, base)


def test_block_dim_sizes_the_grid_only_on_request(R, executor, tmp_path, monkeypatch):
    """AFIR_HIP_HONOUR_BLOCK_DIM=1 makes a positive block_dim the number of workgroups; a run
    manifest says the same with "hip_grid", and the session reports the grid that ran."""
    _, binary = _compile(R, tmp_path, "fused_add_mul")
    a, b = O.gen_c1((300, 1000))
    tiling = R.TilingSchema.for_kernel("fused_add_mul").pack(dim_arg0_0=300, dim_arg0_1=1000)
    out = np.empty_like(a)
    executor.execute(binary, "fused_add_mul", [a, b], [out], tiling, block_dim=8)
    auto = executor.runtime.last_launch()
    assert auto["workgroups"] > 8
    monkeypatch.setenv("AFIR_HIP_HONOUR_BLOCK_DIM", "1")
    executor.execute(binary, "fused_add_mul", [a, b], [out], tiling, block_dim=8)
    assert executor.runtime.last_launch()["workgroups"] == 8
    assert out.tobytes() == O.golden_c1(a, b).tobytes()
    executor.execute(binary, "fused_add_mul", [a, b], [out], tiling, block_dim=0)
    assert executor.runtime.last_launch()["workgroups"] == auto["workgroups"]
    monkeypatch.delenv("AFIR_HIP_HONOUR_BLOCK_DIM")

    src = _descriptor(tmp_path, "fused_add_mul")
    art = tmp_path / "artifact"
    assert _rs("--kernel", str(src), "--output", str(art), "--name", "k").returncode == 0
    np.save(tmp_path / "a.npy", a)
    np.save(tmp_path / "b.npy", b)
    np.save(tmp_path / "e.npy", O.golden_c1(a, b))
    (tmp_path / "ts.json").write_text(json.dumps(
        {"tiling_params": [{"name": "dim_arg0_0"}, {"name": "dim_arg0_1"}]}))
    m = {"task_id": "main", "backend": "hip", "artifact_root": str(art),
         "inputs": [{"name": "a", "path": str(tmp_path / "a.npy")},
                    {"name": "b", "path": str(tmp_path / "b.npy")}],
         "outputs": [{"name": "o", "path": str(tmp_path / "o.npy")}],
         "expected_outputs": [{"name": "o", "path": str(tmp_path / "e.npy")}],
         "tiling": {"schema": str(tmp_path / "ts.json"), "params": "dim_arg0_0=300,dim_arg0_1=1000"},
         "block_dim": 40, "atol": 0, "rtol": 0}
    (tmp_path / "m.json").write_text(json.dumps(m))
    p = _rs("--run-manifest", str(tmp_path / "m.json"), "--run")
    assert p.returncode == 0, p.stdout + p.stderr
    assert "session.runtime.attribute.grid_source=launcher" in p.stdout
    assert f"session.runtime.attribute.grid={auto['workgroups']}x{auto['threads']}" in p.stdout
    assert "session.runtime.counter.block_dim=40" in p.stdout
    m["hip_grid"] = 24
    (tmp_path / "m.json").write_text(json.dumps(m))
    p = _rs("--run-manifest", str(tmp_path / "m.json"), "--run")
    assert p.returncode == 0, p.stdout + p.stderr
    assert "session.runtime.attribute.grid_source=hip_grid" in p.stdout
    assert "session.runtime.attribute.grid=24x" in p.stdout


def test_an_executor_keeps_what_a_repeated_run_needs(R, executor, tmp_path):
    """The same compiled region run again and again on one executor: the program stays registered
    with its code object loaded, so from the second run on the reported kernel time is the
    kernel's (microseconds), not the loading of the code object (hundreds of microseconds), and
    the results stay right with the device buffers reused.  A code object that changes on disk
    is not served from what was kept."""
    import struct
    import time
    from oracle import region_oracle as RO
    from tests import mlir_cases as MC
    from tests import region_cases as RC
    src = tmp_path / "rowsum.mlir"
    src.write_text(MC.ROW_BIAS_REDUCE)
    path = R.compile_kernel(src, tmp_path / "art_rowsum", "k")
    binary = R.read_binary(path)
    assert "code_object=k.hsaco" in binary.decode()
    m, n = 640, 512
    tiling = struct.pack("<4q", m, m, n, m)
    times = []
    for rep in range(4):
        _, (a, b), want = RC.case_reduce_rowbias(m, n, seed=rep)
        out = np.zeros(m, np.float16)
        t = time.perf_counter()
        executor.execute(binary, "k", [a, b], [out], tiling)
        times.append(time.perf_counter() - t)
        assert np.abs(out.view(np.int16).astype(int) - want.view(np.int16).astype(int)).max() <= 1, rep
        assert executor.runtime.last_launch()["kernel_ns"] < 100_000, (rep, executor.runtime.last_launch())
    assert min(times[1:]) < 0.5e-3, times          # 0.76 ms per run before anything was kept
    # the artifact is compiled again (other emit options): same path, another file
    hsaco = tmp_path / "art_rowsum" / "k.hsaco"
    hsaco.write_bytes(b"\x7fELF" + b"\0" * 100)
    with pytest.raises(R.ExecutorError, match="code object"):
        executor.execute(binary, "k", [a, b], [np.zeros(m, np.float16)], tiling)
