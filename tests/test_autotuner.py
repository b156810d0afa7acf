"""Host-side checks of the autotuner CLI: reading a tiling space in the
reference's format (tools/autotuner/autotuner_main.cpp:28-50 flags, :348-470
space parsing), enumerating candidates, and the keys of best_config.json
(:557-595).  The testing driver stands in for the GPU: it runs nothing and
reports a kernel time that falls as block_dim grows."""
import json
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
AT = os.path.join(ROOT, "ascend-mlir_amd", "bin", "autotuner")

from mlir_cases import ROW_BIAS_REDUCE  # noqa: E402


def _at(*args):
    return subprocess.run([AT, *args], capture_output=True, text=True)


def _setup(tmp_path, space):
    (tmp_path / "k.mlir").write_text(ROW_BIAS_REDUCE)
    np.save(tmp_path / "a.npy", np.ones(8, np.float16))
    np.save(tmp_path / "b.npy", np.ones((8, 32), np.float16))
    np.save(tmp_path / "e.npy", np.zeros(8, np.float16))
    (tmp_path / "space.json").write_text(json.dumps(space))
    return ["--space", str(tmp_path / "space.json"), "--kernel", str(tmp_path / "k.mlir"),
            "--inputs", f"{tmp_path / 'a.npy'},{tmp_path / 'b.npy'}", "--expected", str(tmp_path / "e.npy"),
            "--output", str(tmp_path / "best.json"), "--build-dir", str(tmp_path / "art"),
            "--testing-driver=hip-success"]


DIMS = [{"name": "dim_arg0_0", "type": "int64", "fixed": True, "shape_key": "M"},
        {"name": "dim_arg1_0", "type": "int64", "fixed": True, "shape_key": "M"},
        {"name": "dim_arg1_1", "type": "int64", "fixed": True, "shape_key": "N"},
        {"name": "dim_arg2_0", "type": "int64"}]          # taken from e.npy


def test_block_dim_candidates_and_best_config(tmp_path):
    space = {"kernel": "rowbias_reduce", "kernel_file": "k.mlir", "soc": "gfx950",
             "block_dim_values": [0, 64, 256, 128], "tiling_params": DIMS}
    p = _at(*_setup(tmp_path, space), "--shape", "M=8,N=32", "--repeats", "2")
    assert p.returncode == 0, p.stderr + p.stdout
    lines = [l for l in p.stdout.splitlines() if l.startswith("[")]
    assert len(lines) == 4 and lines[0].startswith("[1/4] block_dim=0 ...") and all(" OK " in l for l in lines)
    best = json.loads((tmp_path / "best.json").read_text())
    # every key the reference writes
    for key in ("kernel_name", "kernel_type", "soc", "artifact_root", "manifest_path", "device_binary_path",
                "kernel_file", "best", "config", "shape"):
        assert key in best, key
    assert set(best["best"]) >= {"block_dim", "cycle_count", "score", "max_abs_diff"}
    assert best["best"]["block_dim"] == 256               # the testing driver's fastest
    assert best["kernel_name"] == "rowbias_reduce" and best["soc"] == "gfx950"
    assert best["kernel_file"] == "k.mlir" and best["shape"] == {"M": 8, "N": 32}
    assert best["config"] == {"dim_arg0_0": 8, "dim_arg1_0": 8, "dim_arg1_1": 32, "dim_arg2_0": 8}
    assert best["candidates"] == 4
    assert os.path.exists(best["manifest_path"]) and os.path.exists(best["device_binary_path"])


def test_search_parameters_and_block_dim_expr(tmp_path):
    # a searched parameter in both notations; block_dim follows from it
    space = {"block_dim_expr": "ceil(M / tile_m)",
             "tiling_params": [{"name": "tile_m", "type": "int64", "values": [1, 2, 4]},
                               {"name": "tile_n", "type": "int32", "min": 16, "max": 32, "step": 16},
                               {"name": "m", "type": "int64", "fixed": True, "shape_key": "M"}]}
    p = _at(*_setup(tmp_path, space), "--shape", "M=8,N=32")
    assert p.returncode == 0, p.stderr + p.stdout
    lines = [l for l in p.stdout.splitlines() if l.startswith("[")]
    assert len(lines) == 6
    assert any("tile_m=1" in l and "tile_n=32" in l and "block_dim=8 " in l for l in lines)
    assert any("tile_m=4" in l and "block_dim=2 " in l for l in lines)
    best = json.loads((tmp_path / "best.json").read_text())
    assert best["best"]["block_dim"] == 8 and best["config"]["tile_m"] == 1 and best["config"]["m"] == 8


def test_bad_invocations(tmp_path):
    base = _setup(tmp_path, {"tiling_params": DIMS})
    assert _at().returncode == 4
    assert _at(*base).returncode == 4                                    # --shape missing
    p = _at(*base, "--shape", "M=8")                                     # N missing
    assert p.returncode == 4 and "shape key 'N'" in p.stderr
    p = _at(*base, "--shape", "M=8,N=32", "--artifact-root", str(tmp_path / "art"))
    assert p.returncode == 4 and "exactly one" in p.stderr
    (tmp_path / "space.json").write_text(json.dumps({"tiling_params": [{"name": "tile"}]}))
    p = _at(*base, "--shape", "M=8,N=32")
    assert p.returncode == 4 and "no shape_key, value or candidates" in p.stderr
    (tmp_path / "space.json").write_text(json.dumps(
        {"block_dim_expr": "ceil(M / nope)", "tiling_params": DIMS}))
    p = _at(*base, "--shape", "M=8,N=32")
    assert p.returncode == 4 and "unknown name 'nope'" in p.stderr
    (tmp_path / "space.json").write_text("[1, 2]")
    assert _at(*base, "--shape", "M=8,N=32").returncode == 4


def test_emit_parameters_compile_one_artifact_per_candidate(tmp_path):
    """emit_* parameters are compile-time choices of the emitted kernels: every
    combination gets its own artifact and stays out of the TilingData bytes."""
    from tests import region_cases as RC
    (tmp_path / "k.region").write_text(RC.C3_RELU_BCAST_TRANSPOSE)
    np.save(tmp_path / "x.npy", np.ones((2, 64, 128), np.float16))
    np.save(tmp_path / "c.npy", np.ones((128,), np.float16))
    np.save(tmp_path / "e.npy", np.zeros((2, 128, 64), np.float16))
    space = {"kernel": "c3", "kernel_file": "k.region", "block_dim_values": [0, 8],
             "tiling_params": [{"name": "emit_tile_q", "values": [64, 128]},
                               {"name": "emit_tile_p", "value": 32},
                               {"name": "dim_arg0_0"}, {"name": "dim_arg0_1"}, {"name": "dim_arg0_2"},
                               {"name": "dim_arg1_0"},
                               {"name": "dim_arg2_0"}, {"name": "dim_arg2_1"}, {"name": "dim_arg2_2"}]}
    (tmp_path / "space.json").write_text(json.dumps(space))
    p = _at("--space", str(tmp_path / "space.json"), "--kernel", str(tmp_path / "k.region"),
            "--inputs", f"{tmp_path / 'x.npy'},{tmp_path / 'c.npy'}", "--expected", str(tmp_path / "e.npy"),
            "--shape", "B=2", "--output", str(tmp_path / "best.json"), "--build-dir", str(tmp_path / "art"),
            "--testing-driver=hip-success")
    assert p.returncode == 0, p.stderr + p.stdout
    lines = [l for l in p.stdout.splitlines() if l.startswith("[")]
    assert len(lines) == 4 and all(" OK " in l for l in lines)
    for tq in (64, 128):
        src = (tmp_path / "art" / f"emit_tile_p32_tile_q{tq}" / "c3.hip").read_text()
        assert f"tiles of 32 (dim 1) x {tq} (dim 2)" in src
        assert (tmp_path / "art" / f"emit_tile_p32_tile_q{tq}" / "c3.hsaco").stat().st_size > 0
    best = json.loads((tmp_path / "best.json").read_text())
    assert best["config"]["emit_tile_p"] == 32 and best["config"]["emit_tile_q"] in (64, 128)
    assert best["artifact_root"].endswith(f"emit_tile_p32_tile_q{best['config']['emit_tile_q']}")
    # a choice the emitter refuses fails that candidate only
    space["tiling_params"][0]["values"] = [64, 100]
    (tmp_path / "space.json").write_text(json.dumps(space))
    p = _at("--space", str(tmp_path / "space.json"), "--kernel", str(tmp_path / "k.region"),
            "--inputs", f"{tmp_path / 'x.npy'},{tmp_path / 'c.npy'}", "--expected", str(tmp_path / "e.npy"),
            "--shape", "B=2", "--output", str(tmp_path / "best.json"), "--build-dir", str(tmp_path / "art2"),
            "--testing-driver=hip-success")
    assert p.returncode == 0 and p.stdout.count(" FAIL ") == 2 and "tile_q must be 64, 128 or 256" in p.stdout


def test_build_parameters_stay_out_of_the_tiling_bytes(tmp_path):
    """build_<MACRO> parameters choose a variant of the hand-tuned kernel library; like emit_*
    they are enumerated with the rest of the space and never reach the TilingData bytes.  The
    testing driver builds nothing."""
    space = {"block_dim_values": [0],
             "tiling_params": [{"name": "build_AFIR_ROWSUM_WG_PER_CU", "values": [1, 2, 4]}, *DIMS]}
    p = _at(*_setup(tmp_path, space), "--shape", "M=8,N=32", "--buffer-sets", "3")
    assert p.returncode == 0, p.stderr + p.stdout
    lines = [l for l in p.stdout.splitlines() if l.startswith("[")]
    assert len(lines) == 3 and all(" OK " in l for l in lines)
    assert [l.split()[1] for l in lines] == [f"build_AFIR_ROWSUM_WG_PER_CU={v}" for v in (1, 2, 4)]
    best = json.loads((tmp_path / "best.json").read_text())
    assert best["config"]["build_AFIR_ROWSUM_WG_PER_CU"] in (1, 2, 4)
    assert {k: v for k, v in best["config"].items() if not k.startswith("build_")} == \
        {"dim_arg0_0": 8, "dim_arg1_0": 8, "dim_arg1_1": 32, "dim_arg2_0": 8}


def test_kernel_library_variant_builds_only_what_the_macro_touches(tmp_path):
    """build.py --variant: the library a build_* candidate loads.  Only the sources that
    mention the macro are recompiled; the result exports the launchers of the ordinary library
    and finds the families' code objects beside it."""
    import ctypes
    import sys
    out = tmp_path / "variant_AFIR_ELTWISE_UNROLL4.so"
    p = subprocess.run([sys.executable, os.path.join(ROOT, "ascend-mlir_amd", "build.py"), "--variant", str(out),
                        "-DAFIR_ELTWISE_UNROLL=4"], capture_output=True, text=True)
    assert p.returncode == 0, p.stderr + p.stdout
    assert sorted(os.listdir(tmp_path / "obj_AFIR_ELTWISE_UNROLL-4")) == ["kernels_eltwise.hip.o"]
    assert os.path.isdir(tmp_path / "families")
    lib = ctypes.CDLL(str(out))
    for sym in ("afir_hip_launch_fused_add_mul", "afir_hip_launch_region", "afir_hip_launch_matmul_add_leakyrelu"):
        assert hasattr(lib, sym), sym
    bad = subprocess.run([sys.executable, os.path.join(ROOT, "ascend-mlir_amd", "build.py"), "--variant", str(out),
                          "AFIR_ELTWISE_UNROLL=4"], capture_output=True, text=True)
    assert bad.returncode != 0 and "usage" in bad.stderr


def test_env_parameters_are_set_for_their_candidate_only(tmp_path):
    """env_<NAME>: a launch-time choice the kernels read from the environment (the holds of the
    kernels that separate reads from writes).  The candidate runs with NAME set, the value is
    not part of the tiling bytes, and best_config.json records the winner."""
    space = {"block_dim_values": [0],
             "tiling_params": DIMS + [{"name": "env_AFIR_TESTING_EXTRA_US", "type": "int64", "values": [30, 10, 20]}]}
    p = _at(*_setup(tmp_path, space), "--shape", "M=8,N=32", "--repeats", "2")
    assert p.returncode == 0, p.stderr + p.stdout
    lines = [l for l in p.stdout.splitlines() if l.startswith("[")]
    assert len(lines) == 3
    # the testing driver adds the variable's value (us) to its fixed 1000 us at block_dim 0
    assert [l.split("score=")[1].split()[0] for l in lines] == ["1030000", "1010000", "1020000"]
    best = json.loads((tmp_path / "best.json").read_text())
    assert best["config"]["env_AFIR_TESTING_EXTRA_US"] == 10 and best["best"]["score"] == 1010000
    bad = dict(space, tiling_params=DIMS + [{"name": "env_BAD-NAME", "type": "int64", "values": [1]}])
    p = _at(*_setup(tmp_path, bad), "--shape", "M=8,N=32")
    assert p.returncode == 4 and "variable names" in p.stderr
