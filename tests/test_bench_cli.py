"""bench.py's command line: what it prints and how it refuses."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BENCH = os.path.join(ROOT, "bench.py")


def test_more_than_one_gpu_is_refused_with_a_message():
    p = subprocess.run([sys.executable, BENCH, "--gpus", "2"], capture_output=True, text=True)
    assert p.returncode != 0
    assert "--gpus must be 1" in (p.stdout + p.stderr)


def test_without_a_gpu_it_fails_loudly():
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is visible")
    p = subprocess.run([sys.executable, BENCH, "--steps", "1", "--warmup", "0"], capture_output=True, text=True)
    assert p.returncode != 0
    assert "no CPU fallback" in (p.stdout + p.stderr)
    assert not any(l.startswith("{") for l in p.stdout.splitlines())       # no result line without a measurement


@pytest.mark.gpu
def test_result_line_has_the_agreed_fields():
    p = subprocess.run([sys.executable, BENCH, "--steps", "5", "--warmup", "2", "--no-all", "--no-power-evidence"],
                       capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stderr
    lines = [l for l in p.stdout.splitlines() if l.startswith("{")]
    assert len(lines) == 1
    d = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in d, key
    assert d["n_gpus"] == 1 and d["steps"] == 5 and d["warmup"] == 2 and d["vs_baseline"] is None
    assert d["higher_is_better"] is True and "workload" in d["config"] and "model" not in d["config"]
    r = d["roofline"]
    assert set(("bound", "achieved", "peak", "unit", "frac", "traffic")) <= set(r)
    assert r["bound"] in ("hbm", "mfma") and abs(r["frac"] - r["achieved"] / r["peak"]) < 1e-3 and 0 < r["frac"] < 1
    c = d["cpu_baseline"]
    assert set(("value", "unit", "cores", "kind", "sample")) <= set(c) and c["kind"] in ("port", "reference")
    assert d["parity"]["passed"] is True
