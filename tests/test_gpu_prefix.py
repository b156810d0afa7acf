"""Programs of a hand-tuned family's form launched on the leading part of wider
tensors: the family kernels (dense operands only) must not take such launches;
the result has to match the region oracle on every route."""
import numpy as np
import pytest

from oracle import region_oracle as RO
from tests import prefix_cases as PC

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def H(pkg):
    import torch
    from ascend_mlir_amd import hip_kernels
    hip_kernels.load()
    assert torch.cuda.is_available()
    return hip_kernels


@pytest.fixture(scope="module")
def cache(tmp_path_factory):
    return str(tmp_path_factory.mktemp("prefix_cache"))


def check(got, want, text, inputs):
    if "reduce sum" in text:      # a float32 sum in another order
        x = inputs[0].astype(np.float64)[:, :inputs[1].shape[0]] + inputs[1].astype(np.float64)
        tol = 1e-5 * np.abs(want.astype(np.float64)) + 1e-6 * np.abs(x).sum(axis=1)
        assert np.all(np.abs(got.astype(np.float64) - want.astype(np.float64)) <= tol)
    else:
        assert got.tobytes() == want.tobytes()


@pytest.mark.parametrize("compiled", [False, True], ids=["interpreter", "compiled"])
@pytest.mark.parametrize("which", ["exact", "prefix"])
@pytest.mark.parametrize("name", sorted(PC.CASES))
def test_family_shaped_programs_on_dense_and_prefix_operands(H, cache, monkeypatch, name, which, compiled):
    import torch
    monkeypatch.delenv("AFIR_HIP_REGION_GENERIC", raising=False)
    text, family, exact, prefix = PC.CASES[name]
    shapes = exact if which == "exact" else prefix
    inputs = PC.make_inputs(text, shapes)
    want = RO.evaluate(text, inputs, out_shape=shapes[-1])
    r = H.Region(text)
    try:
        if compiled:
            r.compile(cache_dir=cache)
        tiling = H.pack_tiling(*PC.dims(*shapes))
        assert r.route(tiling) == ("family" if which == "exact" else "compiled" if compiled else "interpreter")
        dev = [torch.from_numpy(x).cuda() for x in inputs]
        out = r(*dev, out_shape=shapes[-1])
        check(out.cpu().numpy(), want, text, inputs)
    finally:
        r.close()
