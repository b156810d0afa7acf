"""The autotuner on a real GPU: every candidate is launched, validated against
the expected output and scored by its measured kernel time
(reference flow: tools/autotuner/autotuner_main.cpp:700-860)."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
from mlir_cases import ROW_BIAS_REDUCE  # noqa: E402

AT = os.path.join(ROOT, "ascend-mlir_amd", "bin", "autotuner")
pytestmark = pytest.mark.gpu

SPACE = {"kernel": "rowbias_reduce", "kernel_file": "k.mlir", "soc": "gfx950",
         "block_dim_values": [0, 256, 1024, 4096],
         "tiling_params": [{"name": "dim_arg0_0", "fixed": True, "shape_key": "M"},
                           {"name": "dim_arg1_0", "fixed": True, "shape_key": "M"},
                           {"name": "dim_arg1_1", "fixed": True, "shape_key": "N"},
                           {"name": "dim_arg2_0", "fixed": True, "shape_key": "M"}]}


def _run(tmp_path, expected, *extra):
    (tmp_path / "k.mlir").write_text(ROW_BIAS_REDUCE)
    (tmp_path / "space.json").write_text(json.dumps(SPACE))
    np.save(tmp_path / "e.npy", expected)
    return subprocess.run(
        [AT, "--space", str(tmp_path / "space.json"), "--kernel", str(tmp_path / "k.mlir"),
         "--inputs", f"{tmp_path / 'a.npy'},{tmp_path / 'b.npy'}", "--expected", str(tmp_path / "e.npy"),
         "--shape", "M=2048,N=1024", "--output", str(tmp_path / "best.json"),
         "--build-dir", str(tmp_path / "art"), *extra], capture_output=True, text=True, timeout=110)


def test_autotune_row_bias_reduce(tmp_path):
    rng = np.random.default_rng(5)
    a = rng.standard_normal(2048).astype(np.float16)
    b = rng.standard_normal((2048, 1024)).astype(np.float16)
    np.save(tmp_path / "a.npy", a)
    np.save(tmp_path / "b.npy", b)
    want = (a[:, None].astype(np.float32) + b.astype(np.float32)).sum(axis=1).astype(np.float16)
    p = _run(tmp_path, want, "--atol", "0.25", "--rtol", "0.01")
    assert p.returncode == 0, p.stdout + p.stderr
    lines = [l for l in p.stdout.splitlines() if l.startswith("[")]
    assert len(lines) == 4 and all(" OK " in l for l in lines), p.stdout
    best = json.loads((tmp_path / "best.json").read_text())
    assert best["best"]["block_dim"] in (0, 256, 1024, 4096)
    assert 0 < best["best"]["score"] < 5_000_000          # ns: a 4 MiB pass takes microseconds
    assert best["best"]["max_abs_diff"] <= 0.25
    scores = [float(l.split("score=")[1].split()[0]) for l in lines]
    assert best["best"]["score"] == round(min(scores))

    # an expected output no candidate can match: every candidate FAILs, exit 1
    p = _run(tmp_path, want + np.float16(3.0), "--atol", "0.25", "--rtol", "0.01")
    assert p.returncode == 1, p.stdout + p.stderr
    assert p.stdout.count(" FAIL ") == 4 and "no candidate passed" in p.stderr


def test_autotune_tile_shapes_of_a_transposing_region(tmp_path):
    """Tile shapes as searched parameters: each candidate is compiled, run and
    validated bit-exactly (atol = rtol = 0) against the oracle's result."""
    from tests import region_cases as RC
    from oracle import region_oracle as RO
    rng = np.random.default_rng(9)
    x = rng.standard_normal((3, 200, 136)).astype(np.float16)       # ragged against every tile shape
    c = rng.standard_normal((136,)).astype(np.float16)
    want = RO.evaluate(RC.C3_RELU_BCAST_TRANSPOSE, [x, c])
    (tmp_path / "k.region").write_text(RC.C3_RELU_BCAST_TRANSPOSE)
    np.save(tmp_path / "x.npy", x)
    np.save(tmp_path / "c.npy", c)
    np.save(tmp_path / "e.npy", want)
    space = {"kernel": "c3", "kernel_file": "k.region", "block_dim_values": [0],
             "tiling_params": [{"name": "emit_tile_p", "values": [32, 64]}, {"name": "emit_tile_q", "values": [64, 128]},
                               {"name": "dim_arg0_0"}, {"name": "dim_arg0_1"}, {"name": "dim_arg0_2"}, {"name": "dim_arg1_0"},
                               {"name": "dim_arg2_0"}, {"name": "dim_arg2_1"}, {"name": "dim_arg2_2"}]}
    (tmp_path / "space.json").write_text(json.dumps(space))
    p = subprocess.run([AT, "--space", str(tmp_path / "space.json"), "--kernel", str(tmp_path / "k.region"),
                        "--inputs", f"{tmp_path / 'x.npy'},{tmp_path / 'c.npy'}", "--expected", str(tmp_path / "e.npy"),
                        "--shape", "B=3", "--output", str(tmp_path / "best.json"), "--build-dir", str(tmp_path / "art"),
                        "--atol", "0", "--rtol", "0"], capture_output=True, text=True, timeout=110)
    assert p.returncode == 0, p.stdout + p.stderr
    lines = [l for l in p.stdout.splitlines() if l.startswith("[")]
    assert len(lines) == 4 and all(" OK " in l and "max_abs_diff=0" in l for l in lines), p.stdout
    best = json.loads((tmp_path / "best.json").read_text())
    assert (best["config"]["emit_tile_p"], best["config"]["emit_tile_q"]) in [(32, 64), (32, 128), (64, 64), (64, 128)]


def test_rotating_buffer_sets_and_ramp(tmp_path):
    """--buffer-sets N: the timed launches rotate over N device copies of the tensors; --ramp-ms:
    a candidate is launched back to back before it is timed and scored by the average of its
    timed launches.  The output handed back (and validated) is that of the first copy; the score
    stays a positive kernel time."""
    rng = np.random.default_rng(6)
    a = rng.standard_normal(2048).astype(np.float16)
    b = rng.standard_normal((2048, 1024)).astype(np.float16)
    np.save(tmp_path / "a.npy", a)
    np.save(tmp_path / "b.npy", b)
    want = (a[:, None].astype(np.float32) + b.astype(np.float32)).sum(axis=1).astype(np.float16)
    p = _run(tmp_path, want, "--atol", "0.25", "--rtol", "0.01", "--buffer-sets", "3", "--ramp-ms", "5",
             "--repeats", "24")
    assert p.returncode == 0, p.stdout + p.stderr
    lines = [l for l in p.stdout.splitlines() if l.startswith("[")]
    assert len(lines) == 4 and all(" OK " in l for l in lines), p.stdout
    scores = [float(l.split("score=")[1].split()[0]) for l in lines]
    assert all(0 < s < 5_000_000 for s in scores)
    best = json.loads((tmp_path / "best.json").read_text())
    assert best["best"]["score"] == round(min(scores)) and best["best"]["max_abs_diff"] <= 0.25
    # a wrong expectation still fails every candidate: the rotation does not hide the first copy's output
    p = _run(tmp_path, want + np.float16(3.0), "--atol", "0.25", "--rtol", "0.01", "--buffer-sets", "3",
             "--ramp-ms", "5", "--repeats", "8")
    assert p.returncode == 1 and p.stdout.count(" FAIL ") == 4
