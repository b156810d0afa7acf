"""The GPU path on the reference's own vectors (inputs and expected outputs
written by the reference's golden scripts, tests/golden/reference_examples.npz):
MLIR graph -> region program -> kernel, compared with the reference's output.
Needs a GPU."""
import os
import subprocess

import numpy as np
import pytest

from tests import golden_cases as GC

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TR = os.path.join(ROOT, "ascend-mlir_amd", "bin", "afir-translate")
CASES = list(GC.cases())


@pytest.mark.parametrize("generic", ["routed", "generic", "compiled"])
@pytest.mark.parametrize("case", CASES, ids=[c[0] for c in CASES])
def test_kernel_reproduces_the_reference_output(pkg, monkeypatch, tmp_path_factory, case, generic):
    import torch
    from ascend_mlir_amd import hip_kernels as H
    H.load()
    name, mlir, program, inputs, want, exact = case
    if program is None:
        p = subprocess.run([TR, "-mlir-to-hip", "-"], input=mlir, capture_output=True, text=True)
        assert p.returncode == 0, p.stderr
        program = p.stdout
    monkeypatch.setenv("AFIR_HIP_REGION_GENERIC", "0" if generic == "routed" else "1")
    r = H.Region(program)
    if generic == "compiled" and "matmul" not in program:
        r.compile(cache_dir=str(tmp_path_factory.mktemp("region_cache")))
        assert r.kernel == "fused_region_compiled"
    dev = [torch.from_numpy(x).cuda() for x in inputs]
    got = r(*dev, out_shape=want.shape).cpu().numpy()
    r.close()
    if exact:
        assert got.tobytes() == want.tobytes()
    else:   # f32 row sum in another order, one rounding to f16
        assert np.all(np.abs(got.astype(np.float64) - want.astype(np.float64))
                      <= 2.0 ** -10 * np.abs(want.astype(np.float64)) + 1e-3)


@pytest.mark.parametrize("generic", ["routed", "generic", "compiled"])
def test_mean_kernel_agrees_with_the_reference_sum_vector(pkg, monkeypatch, tmp_path_factory, generic):
    import torch
    from ascend_mlir_amd import hip_kernels as H
    H.load()
    mlir, inputs, want = GC.mean_case()
    p = subprocess.run([TR, "-mlir-to-hip", "-"], input=mlir, capture_output=True, text=True)
    assert p.returncode == 0, p.stderr
    monkeypatch.setenv("AFIR_HIP_REGION_GENERIC", "0" if generic == "routed" else "1")
    r = H.Region(p.stdout)
    if generic == "compiled":
        r.compile(cache_dir=str(tmp_path_factory.mktemp("region_cache")))
        assert r.kernel == "fused_region_compiled"
    got = r(*[torch.from_numpy(x).cuda() for x in inputs], out_shape=want.shape).cpu().numpy()
    r.close()
    # sum in another order, then the division: one ulp for each
    g, w = got.astype(np.float64), want.astype(np.float64)
    assert np.all(np.abs(g - w) <= 2.0 ** -9 * np.abs(w) + 1e-5)
