"""Host-side runtime: formats, C API error behaviour, CLI contract.  CPU only."""
import ctypes
import json
import os
import re
import struct
import subprocess

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "ascend-mlir_amd")
RS = os.path.join(PKG, "bin", "runtime-session")

EXAMPLE_MLIR = """func.func @example(%arg0: tensor<4x4xf32>, %arg1: tensor<4x4xf32>) -> tensor<4x4xf32> {
  %0 = afir.add %arg0, %arg1 : (tensor<4x4xf32>, tensor<4x4xf32>) -> tensor<4x4xf32>
  %1 = afir.mul %0, %arg1 : (tensor<4x4xf32>, tensor<4x4xf32>) -> tensor<4x4xf32>
  return %1 : tensor<4x4xf32>
}
"""


def test_cpp_host_tests(tmp_path):
    exe = tmp_path / "test_runtime_host"
    src = [os.path.join(ROOT, "tests", "cpp", "test_runtime_host.cpp"),
           os.path.join(PKG, "csrc", "runtime", "support.cpp"),
           os.path.join(PKG, "csrc", "runtime", "artifact.cpp"),
           os.path.join(PKG, "csrc", "runtime", "session.cpp"),
           os.path.join(PKG, "csrc", "target", "region_program.cpp"),
           os.path.join(PKG, "csrc", "target", "hip_emitter.cpp"), os.path.join(PKG, "csrc", "target", "hiprtc_compile.cpp"),
           os.path.join(PKG, "csrc", "target", "mlir_translate.cpp")]
    subprocess.run(["g++", "-std=c++17", "-O1", "-Wall", "-I", os.path.join(PKG, "csrc", "runtime"),
                    "-I", os.path.join(ROOT, "include"), *src, "-ldl", "-o", str(exe)], check=True)
    work = tmp_path / "w"
    work.mkdir()
    p = subprocess.run([str(exe), str(work)], capture_output=True, text=True)
    assert p.returncode == 0, p.stdout + p.stderr
    assert " 0 failed" in p.stdout


def _declared(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(afirt_[a-z_]+)\s*\(", text)))


def test_capi_exports_every_declared_symbol(pkg):
    from ascend_mlir_amd.runtime import capi
    L = capi.load_capi()
    names = _declared("afirt_runtime.h")
    assert sorted(capi.EXPORTED_SYMBOLS) == names
    for n in names:
        assert hasattr(L, n), n


def test_capi_error_behaviour_without_gpu(pkg, tmp_path):
    from ascend_mlir_amd.runtime import capi
    L = capi.load_capi()
    err = ctypes.create_string_buffer(256)
    # null / uninitialised handles are errors, not crashes
    assert L.afirt_executor_initialize(None, 0, err, len(err)) == 1
    assert err.value == b"executor handle is null"
    h = L.afirt_executor_create()
    assert h
    assert L.afirt_executor_initialize(h, -1, err, len(err)) == 1
    assert err.value == b"device id must be non-negative"
    vp, sz = ctypes.c_void_p, ctypes.c_size_t
    ptrs, sizes = (vp * 1)(0), (sz * 1)(0)
    rc = L.afirt_executor_run(h, None, 0, b"k", 0, ptrs, sizes, 1, ptrs, sizes, None, 0, 1,
                              capi.MAGIC_ELF_AIVEC, err, len(err))
    assert rc == 1 and err.value == b"executor has not been initialized"
    rc = L.afirt_executor_run_file(h, b"/x", b"k", 0, ptrs, sizes, 1, ptrs, sizes, None, 0, 1,
                                   capi.MAGIC_ELF_AIVEC, err, len(err))
    assert rc == 1 and err.value == b"executor has not been initialized"
    # message is truncated into the caller's buffer and NUL-terminated
    small = ctypes.create_string_buffer(8)
    assert L.afirt_executor_initialize(None, 0, small, len(small)) == 1
    assert small.value == b"executo"
    L.afirt_executor_destroy(h)
    # compiler
    buf = ctypes.create_string_buffer(512)
    assert L.afirt_compiler_compile(None, b"a", b"b", b"c", buf, len(buf)) == 1
    assert buf.value == b"compiler handle is null"
    c = L.afirt_compiler_create(b"gfx950", b"gfx950-vec", 3)
    assert L.afirt_compiler_compile(c, b"/no/such/file.mlir", str(tmp_path).encode(), b"k", buf,
                                    len(buf)) == 1
    assert b"cannot read kernel source" in buf.value
    src = tmp_path / "example.mlir"
    src.write_text(EXAMPLE_MLIR)
    assert L.afirt_compiler_compile(c, str(src).encode(), str(tmp_path / "art").encode(), b"example",
                                    buf, len(buf)) == 0
    assert buf.value.decode().endswith("art/example.hipk")
    assert os.path.exists(buf.value.decode())
    bad = tmp_path / "bad.mlir"
    bad.write_text("func.func @unknown_thing() { return }\n")
    assert L.afirt_compiler_compile(c, str(bad).encode(), str(tmp_path / "art2").encode(), b"", buf,
                                    len(buf)) == 1
    assert b"cannot lower kernel source" in buf.value
    L.afirt_compiler_destroy(c)
    L.afirt_compiler_destroy(None)
    L.afirt_executor_destroy(None)


def test_python_runtime_mirror(pkg, tmp_path):
    from ascend_mlir_amd import runtime as R
    src = tmp_path / "k.mlir"
    src.write_text(EXAMPLE_MLIR)
    path = R.compile_kernel(src, tmp_path / "art", "example")
    text = R.read_binary(path).decode()
    assert text.startswith("afir-hip-artifact 1\n") and "hip_kernel=fused_region" in text
    # the AFIR chain became a region program: (arg0 + arg1) * arg1
    program = text.split("\nprogram:\n", 1)[1].split()
    assert program[:3] == ["afir-hip-region", "1", "arg"]
    assert " ".join(program).endswith("push arg0 d0 d1 push arg1 d0 d1 add push arg1 d0 d1 mul store end")
    manifest = (tmp_path / "art" / "out" / "manifest.txt").read_text()
    assert "kernel_name=example" in manifest and "kernel_so_symbol=afir_hip_launch_region" in manifest
    with pytest.raises(R.CompilerError):
        R.compile_kernel(tmp_path / "missing.mlir", tmp_path / "a2", "x")
    ex = R.KernelExecutor()
    with pytest.raises(R.ExecutorError):   # no device in this container
        ex.initialize()


# --- the reference's Python tiling-schema tests, restated --------------------

@pytest.fixture()
def schema_file(tmp_path):
    p = tmp_path / "tiling_space.json"
    p.write_text(json.dumps({"tiling_params": [
        {"name": "TB_M", "type": "int64"}, {"name": "TB_N", "type": "int64"},
        {"name": "M", "type": "int64"}, {"name": "N", "type": "int32"}]}))
    return p


def test_tiling_schema_python(pkg, schema_file, tmp_path):
    from ascend_mlir_amd.runtime import TilingSchema
    s = TilingSchema.from_json(schema_file)
    assert len(s) == 4 and s.field_names == ["TB_M", "TB_N", "M", "N"]
    b = s.pack(TB_M=16, TB_N=4, M=64, N=64)
    assert len(b) == 28 and struct.unpack("<qqqi", b) == (16, 4, 64, 64)
    assert s.pack(N=64, M=64, TB_N=4, TB_M=16) == b          # keyword order is irrelevant
    with pytest.raises(ValueError, match="missing tiling fields"):
        s.pack(TB_M=16)
    with pytest.raises(ValueError, match="unexpected tiling fields"):
        s.pack(TB_M=16, TB_N=4, M=64, N=64, K=1)
    with pytest.raises(FileNotFoundError):
        TilingSchema.from_json(tmp_path / "none.json")
    bad = tmp_path / "bad.json"
    bad.write_text("{ nope")
    with pytest.raises(ValueError, match="JSON parse error"):
        TilingSchema.from_json(bad)
    bad.write_text("{}")
    with pytest.raises(ValueError, match="missing 'tiling_params'"):
        TilingSchema.from_json(bad)
    bad.write_text('{"tiling_params": [{"type": "int64"}]}')
    with pytest.raises(ValueError, match="missing 'name'"):
        TilingSchema.from_json(bad)
    assert TilingSchema.for_kernel("matmul_add_leakyrelu").field_names == [
        "dim_arg0_0", "dim_arg0_1", "dim_arg1_1", "alpha_f32_bits"]


# --- runtime-session CLI contract --------------------------------------------

# TilingData of the compiled example: every dim of every argument (a, b, out)
TILING_FIELDS = ["dim_arg0_0", "dim_arg0_1", "dim_arg1_0", "dim_arg1_1", "dim_arg2_0", "dim_arg2_1"]
TILING_PARAMS = ",".join(f"{n}=4" for n in TILING_FIELDS)


def _rs(*args, cwd=None):
    return subprocess.run([RS, *args], capture_output=True, text=True, cwd=cwd)


def _manifest(tmp_path, expected=True, **over):
    a = np.arange(16, dtype=np.float32).reshape(4, 4)
    np.save(tmp_path / "a.npy", a)
    np.save(tmp_path / "b.npy", np.ones((4, 4), np.float32))
    np.save(tmp_path / "exp.npy", np.zeros((4, 4), np.float32))
    (tmp_path / "ts.json").write_text(json.dumps(
        {"tiling_params": [{"name": n} for n in TILING_FIELDS]}))
    m = {"task_id": "main", "backend": "hip", "artifact_root": str(tmp_path / "art"),
         "inputs": [{"name": "a", "path": str(tmp_path / "a.npy")},
                    {"name": "b", "path": str(tmp_path / "b.npy")}],
         "outputs": [{"name": "out", "path": str(tmp_path / "out.npy")}],
         "tiling": {"schema": str(tmp_path / "ts.json"), "params": TILING_PARAMS},
         "block_dim": 0, "atol": 0, "rtol": 0}
    if expected:
        m["expected_outputs"] = [{"name": "out", "path": str(tmp_path / "exp.npy")}]
    else:
        m["outputs"][0].update({"shape": [4, 4], "dtype": "f32"})
    m.update(over)
    (tmp_path / "m.json").write_text(json.dumps(m))
    return str(tmp_path / "m.json")


def test_cli_compile_plan_and_exit_codes(tmp_path):
    src = tmp_path / "example.mlir"
    src.write_text(EXAMPLE_MLIR)
    p = _rs("--kernel", str(src), "--kernel-kind", "vec", "--output", str(tmp_path / "art"),
            "--name", "example")
    assert p.returncode == 0, p.stderr
    out = p.stdout.splitlines()
    assert "artifact.kernel_name=example" in out and f"artifact.root={tmp_path / 'art'}" in out
    assert "artifact.soc=gfx950" in out and "session.plan.tasks=1" in out and "session.plan[0]=main" in out
    assert _rs("--artifact-root", str(tmp_path / "art")).returncode == 0
    assert _rs().returncode == 4
    assert _rs("--kernel", str(src), "--artifact-root", str(tmp_path / "art")).returncode == 4
    assert _rs("--kernel", str(src), "--kernel-kind", "weird", "--output", str(tmp_path / "x")).returncode == 4
    assert _rs("--run-manifest", str(tmp_path / "none.json"), "--run").returncode == 4
    assert _rs("--artifact-root", str(tmp_path / "nope")).returncode == 4
    assert _rs("--bogus").returncode == 4


def test_cli_run_with_testing_driver(tmp_path):
    src = tmp_path / "example.mlir"
    src.write_text(EXAMPLE_MLIR)
    assert _rs("--kernel", str(src), "--output", str(tmp_path / "art"), "--name", "example").returncode == 0
    m = _manifest(tmp_path)
    p = _rs("--run-manifest", m, "--run", "--testing-driver=hip-success")
    assert p.returncode == 0, p.stderr
    lines = p.stdout.splitlines()
    for want in ("session.backend=hip", "session.result=success", "session.validation=pass",
                 "session.profile.count=0", "session.runtime.counter.tiling_bytes=48"):
        assert want in lines, p.stdout
    assert np.array_equal(np.load(tmp_path / "out.npy"), np.zeros((4, 4), np.float32))
    # no expected outputs: no validation line, shapes come from the output binding
    p = _rs("--run-manifest", _manifest(tmp_path, expected=False), "--run", "--testing-driver=hip-success")
    assert p.returncode == 0 and "session.validation=pass" not in p.stdout
    # validation failure: exit 2, stage 'validate', lines on stderr
    m = _manifest(tmp_path)
    np.save(tmp_path / "exp.npy", np.ones((4, 4), np.float32))
    p = _rs("--run-manifest", m, "--run", "--testing-driver=hip-success")
    assert p.returncode == 2
    err = p.stderr.splitlines()
    assert "session.result=error" in err and "session.validation=fail" in err
    assert "session.error_stage=validate" in err
    assert any(l.startswith("Error: [hip:validate] output comparison failed") for l in err)


def test_cli_error_stages(tmp_path):
    src = tmp_path / "example.mlir"
    src.write_text(EXAMPLE_MLIR)
    assert _rs("--kernel", str(src), "--output", str(tmp_path / "art"), "--name", "example").returncode == 0
    # without a GPU the real runner fails at executor_initialize, and says so
    p = _rs("--run-manifest", _manifest(tmp_path), "--run")
    assert p.returncode == 2
    assert "session.error_stage=executor_initialize" in p.stderr.splitlines()
    # missing input file -> bindings
    m = _manifest(tmp_path, inputs=[{"name": "a", "path": str(tmp_path / "gone.npy")}])
    p = _rs("--run-manifest", m, "--run", "--testing-driver=hip-success")
    assert p.returncode == 2 and "session.error_stage=bindings" in p.stderr
    # tiling params that do not match the schema -> bindings
    m = _manifest(tmp_path, tiling={"schema": str(tmp_path / "ts.json"), "params": "dim_arg0_0=4"})
    p = _rs("--run-manifest", m, "--run", "--testing-driver=hip-success")
    assert p.returncode == 2 and "missing field" in p.stderr
    # bad artifact root -> artifact
    m = _manifest(tmp_path, artifact_root=str(tmp_path / "nowhere"))
    p = _rs("--run-manifest", m, "--run", "--testing-driver=hip-success")
    assert p.returncode == 2 and "session.error_stage=artifact" in p.stderr
    # a manifest written for the reference's simulator still runs, and says what it asked for
    m = _manifest(tmp_path, backend="sim")
    np.save(tmp_path / "exp.npy", np.zeros((4, 4), np.float32))
    p = _rs("--run-manifest", m, "--run", "--testing-driver=hip-success")
    assert p.returncode == 0 and "session.backend_requested=sim" in p.stdout


# --- multi-task manifests: plan order, task-output bindings (CPU, testing driver) ---

def _two_task_manifest(tmp_path, **second):
    src = tmp_path / "example.mlir"
    src.write_text(EXAMPLE_MLIR)
    assert _rs("--kernel", str(src), "--output", str(tmp_path / "art"), "--name", "example").returncode == 0
    np.save(tmp_path / "a.npy", np.zeros((4, 4), np.float32))
    np.save(tmp_path / "b.npy", np.ones((4, 4), np.float32))
    (tmp_path / "ts.json").write_text(json.dumps({"tiling_params": [{"name": n} for n in TILING_FIELDS]}))
    tiling = {"schema": str(tmp_path / "ts.json"), "params": TILING_PARAMS}
    first = {"task_id": "first", "inputs": [{"name": "a", "path": str(tmp_path / "a.npy")},
                                           {"name": "b", "path": str(tmp_path / "b.npy")}],
             "outputs": [{"name": "t", "shape": [4, 4], "dtype": "f32"}], "tiling": tiling}
    then = {"task_id": "then", "dependencies": ["first"],
            "inputs": [{"name": "x", "source": "task_output", "upstream_task": "first", "upstream_output": "t"},
                       {"name": "b", "path": str(tmp_path / "b.npy")}],
            "outputs": [{"name": "y", "path": str(tmp_path / "y.npy"), "shape": [4, 4], "dtype": "f32"}],
            "tiling": tiling}
    then.update(second)
    m = {"backend": "hip", "artifact_root": str(tmp_path / "art"), "tasks": [then, first]}
    (tmp_path / "m.json").write_text(json.dumps(m))
    return str(tmp_path / "m.json")


def test_cli_multi_task_plan_and_task_output_binding(tmp_path):
    m = _two_task_manifest(tmp_path)
    p = _rs("--run-manifest", m)
    assert p.returncode == 0, p.stderr
    lines = p.stdout.splitlines()
    # dependencies first, whatever the order in the file
    assert "session.plan.tasks=2" in lines and "session.plan[0]=first" in lines and "session.plan[1]=then" in lines
    p = _rs("--run-manifest", m, "--run", "--testing-driver=hip-success")
    assert p.returncode == 0, p.stderr
    assert "session.result=success" in p.stdout.splitlines()
    # the intermediate tensor was materialised next to the manifest and fed to the second task
    assert (tmp_path / "first__t.npy").exists() and (tmp_path / "y.npy").exists()
    assert "session.runtime.counter.first.tiling_bytes=48" in p.stdout.splitlines()
    assert "session.runtime.counter.then.tiling_bytes=48" in p.stdout.splitlines()


def test_cli_multi_task_errors(tmp_path):
    m = _two_task_manifest(tmp_path, dependencies=["nowhere"])
    p = _rs("--run-manifest", m)
    assert p.returncode == 4 and "unknown task dependency" in p.stderr
    m = _two_task_manifest(tmp_path, inputs=[{"name": "x", "source": "task_output", "upstream_task": "first",
                                              "upstream_output": "missing"},
                                             {"name": "b", "path": str(tmp_path / "b.npy")}])
    p = _rs("--run-manifest", m, "--run", "--testing-driver=hip-success")
    assert p.returncode == 2 and "cannot resolve upstream output first::missing for task then" in p.stderr
    assert "session.error_stage=bindings" in p.stderr
    m = _two_task_manifest(tmp_path, inputs=[{"name": "x", "source": "task_output", "upstream_task": "first"}])
    assert _rs("--run-manifest", m).returncode == 4
    # a cycle
    d = json.loads(open(_two_task_manifest(tmp_path)).read())
    d["tasks"][1]["dependencies"] = ["then"]
    (tmp_path / "cycle.json").write_text(json.dumps(d))
    p = _rs("--run-manifest", str(tmp_path / "cycle.json"))
    assert p.returncode == 4 and "task graph contains a cycle" in p.stderr
    d["tasks"][1]["dependencies"] = []
    d["tasks"][1]["task_id"] = "then"
    (tmp_path / "dup.json").write_text(json.dumps(d))
    p = _rs("--run-manifest", str(tmp_path / "dup.json"))
    assert p.returncode == 4 and "duplicate task id" in p.stderr


def test_cli_profiling_writes_trace_and_retained_summary(tmp_path):
    """"profiling": true -> trace.json per task (schema version 1 of
    lib/Runtime/Execution/SimBackend.cpp:314-374) and a retained
    session_summary.json (lib/Runtime/Profile/ProfileUtils.cpp:134-345),
    announced on the session.profile.* lines
    (tools/runtime-session/runtime_session_main.cpp:167-177)."""
    src = tmp_path / "example.mlir"
    src.write_text(EXAMPLE_MLIR)
    assert _rs("--kernel", str(src), "--output", str(tmp_path / "art"), "--name", "example").returncode == 0
    m = _manifest(tmp_path, profiling=True, block_dim=3, workspace_size=64)
    tmp = tmp_path / "tmp"
    tmp.mkdir()
    p = subprocess.run([RS, "--run-manifest", m, "--run", "--testing-driver=hip-success"], capture_output=True,
                       text=True, env=dict(os.environ, TMPDIR=str(tmp)))
    assert p.returncode == 0, p.stderr
    kv = dict(l.split("=", 1) for l in p.stdout.splitlines() if "=" in l)
    sid = kv["session.profile.session_id"]
    assert re.fullmatch(r"runtime-session-[a-z0-9]{6}", sid)
    assert kv["session.profile.count"] == "1"
    retained = kv["session.profile[0]"]
    assert retained == str(tmp / "ascendc-runtime-profiles" / sid / "tasks" / "main.json")
    trace = json.loads(open(retained).read())
    assert trace == json.loads((tmp_path / "opprof" / "hip" / "main" / "trace.json").read_text())
    for key in ("schema_version", "backend", "session_id", "task_id", "kernel_name", "kernel_kind", "soc_version",
                "block_dim", "workspace_size", "cycle_count", "elapsed_us", "score", "validation_passed",
                "artifact_root", "inputs", "outputs", "tiling"):
        assert key in trace, key
    assert trace["schema_version"] == 1 and trace["backend"] == "hip" and trace["session_id"] == sid
    assert trace["task_id"] == "main" and trace["kernel_name"] == "example" and trace["kernel_kind"] == "vec"
    assert trace["block_dim"] == 3 and trace["workspace_size"] == 64
    assert trace["score"] == trace["cycle_count"] == 12500 and trace["elapsed_us"] == 13
    assert trace["inputs"] == [{"name": "a", "shape": [4, 4], "dtype": "f32"},
                               {"name": "b", "shape": [4, 4], "dtype": "f32"}]
    assert trace["outputs"] == [{"name": "out", "shape": [4, 4], "dtype": "f32"}]
    assert trace["tiling"]["present"] is True and trace["tiling"]["bytes"] == 48
    assert open(trace["tiling"]["binary_path"], "rb").read() == struct.pack("<6q", *[4] * 6)
    summary = json.loads(open(kv["session.profile.summary"]).read())
    assert summary["schema_version"] == 1 and summary["session_id"] == sid and summary["backend"] == "hip"
    assert summary["task_count"] == summary["successful_task_count"] == 1 and summary["failed_task_count"] == 0
    assert summary["tasks"] == [{"task_id": "main", "profile_path": retained, "score": 12500, "cycle_count": 12500}]
    assert summary["total_score"] == summary["total_cycle_count"] == 12500
    assert summary["runtime"]["counters"]["kernel_ns"] == 12500
    assert summary["runtime"]["attributes"]["kernel_name"] == "example"
    # block_dim is the reference's AI-core count: recorded, never the grid; "hip_grid" is one
    assert kv["session.runtime.counter.block_dim"] == "3"
    assert kv["session.runtime.attribute.grid_source"] == "launcher" and kv["session.runtime.attribute.grid"] == "2048x256"
    p = subprocess.run([RS, "--run-manifest", _manifest(tmp_path, block_dim=40, hip_grid=24), "--run",
                        "--testing-driver=hip-success"], capture_output=True, text=True, env=dict(os.environ, TMPDIR=str(tmp)))
    assert "session.runtime.attribute.grid=24x256" in p.stdout and "session.runtime.attribute.grid_source=hip_grid" in p.stdout
    p = subprocess.run([RS, "--run-manifest", _manifest(tmp_path, hip_grid=-1), "--run", "--testing-driver=hip-success"],
                       capture_output=True, text=True)
    assert p.returncode == 4 and "hip_grid must be between" in p.stderr
    # without "profiling" nothing is written
    p = subprocess.run([RS, "--run-manifest", _manifest(tmp_path), "--run", "--testing-driver=hip-success"],
                       capture_output=True, text=True, env=dict(os.environ, TMPDIR=str(tmp)))
    assert "session.profile.count=0" in p.stdout.splitlines() and "session.profile.summary" not in p.stdout
