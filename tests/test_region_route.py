"""Which kernels a fused-region launch runs on, decided on the host from the
program and the shapes of the launch (afir_hip_region_route).  No GPU needed:
nothing is launched."""
import struct

import pytest

from tests import prefix_cases as PC
from tests import region_cases as RC


@pytest.fixture(scope="module")
def H(pkg):
    from ascend_mlir_amd import hip_kernels
    hip_kernels.load()
    return hip_kernels


def tiling(shapes):
    d = PC.dims(*shapes)
    return struct.pack("<%dq" % len(d), *d)


@pytest.mark.parametrize("name", sorted(PC.CASES))
def test_family_route_needs_dense_operands_of_the_iteration_extents(H, name, monkeypatch):
    monkeypatch.delenv("AFIR_HIP_REGION_GENERIC", raising=False)
    text, family, exact, prefix = PC.CASES[name]
    r = H.Region(text)
    try:
        assert r.kernel == family                     # the program has the family's form
        assert r.route(tiling(exact)) == "family"     # and dense operands reach its kernel
        assert r.route(tiling(prefix)) == "interpreter"   # a prefix of wider tensors does not
    finally:
        r.close()


def test_route_of_programs_outside_the_families(H, monkeypatch):
    monkeypatch.delenv("AFIR_HIP_REGION_GENERIC", raising=False)
    r = H.Region(RC.ADD_MUL_3)
    try:
        assert r.kernel == "fused_region"
        assert r.route(tiling([(33, 77)] * 4)) == "interpreter"
        with pytest.raises(H.AfirHipError):
            r.route(b"\0" * 8)                        # wrong number of tiling bytes
    finally:
        r.close()


def test_extents_of_one_leave_their_stride_free(H, monkeypatch):
    """A single row of a wider tensor is still a dense row."""
    monkeypatch.delenv("AFIR_HIP_REGION_GENERIC", raising=False)
    text, family, _, _ = PC.CASES["rowsum"]
    r = H.Region(text)
    try:
        assert r.route(tiling([(1, 8192), (4096,), (1,)])) == "family"
        assert r.route(tiling([(2, 8192), (4096,), (2,)])) == "interpreter"
    finally:
        r.close()
