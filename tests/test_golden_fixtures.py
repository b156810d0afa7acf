"""The oracle against the reference's own vectors: inputs and expected outputs
written by the reference's golden scripts (tests/golden/reference_examples.npz).
The closed-form goldens of afir_oracle and the region oracle on the translated
graphs must reproduce them bit for bit.  CPU only."""
import os
import subprocess

import numpy as np
import pytest

from oracle import afir_oracle as O
from oracle import region_oracle as RO
from tests import golden_cases as GC

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TR = os.path.join(ROOT, "ascend-mlir_amd", "bin", "afir-translate")
CASES = list(GC.cases())


def test_fixture_is_loadable_without_pickle():
    z = GC.load()
    assert len(z.files) == 30
    assert z["matmul-add-leakyrelu/output"].dtype == np.float32
    assert z["gather-elementwise-fusion/input_indices"].dtype == np.int64


def test_closed_form_goldens_reproduce_the_reference_outputs():
    z = GC.load()
    e = "broadcast-add-reduce/"
    assert O.reduce_rowbias_f16(z[e + "input_a"], z[e + "input_b"]).tobytes() == z[e + "output_c"].tobytes()
    e = "relu-broadcast-transpose/"
    assert O.relu_col_add_f16(z[e + "input_data0"], z[e + "input_data1"]).tobytes() == z[e + "output_expected"].tobytes()
    e = "gather-elementwise-fusion/"
    got = O.relu_colgather_add_f16(z[e + "input_data"], z[e + "input_indices"], z[e + "input_bias"])
    assert np.ascontiguousarray(got).tobytes() == np.ascontiguousarray(z[e + "output_out"]).tobytes()
    e = "matmul-add-leakyrelu/"
    got = O.matmul_bias_leakyrelu_f16(z[e + "input_a"], z[e + "input_b"], z[e + "input_bias"], 0.001)
    assert got.tobytes() == z[e + "output"].tobytes()
    e = "real-npu-microcases/relu_only/"
    assert O.op_relu(z[e + "input"].astype(np.float32)).astype(np.float16).tobytes() == z[e + "expected"].tobytes()


@pytest.mark.parametrize("case", CASES, ids=[c[0] for c in CASES])
def test_translated_graph_evaluates_to_the_reference_output(case):
    name, mlir, program, inputs, want, exact = case
    if program is None:
        p = subprocess.run([TR, "-mlir-to-hip", "-"], input=mlir, capture_output=True, text=True)
        assert p.returncode == 0, p.stderr
        program = p.stdout
    got = RO.evaluate(program, inputs)
    assert got.dtype == want.dtype and got.shape == want.shape
    assert got.tobytes() == want.tobytes()      # numpy pairwise f32 sum in both: the reduce is exact too


def test_mean_graph_agrees_with_the_reference_sum_vector():
    mlir, inputs, want = GC.mean_case()
    p = subprocess.run([TR, "-mlir-to-hip", "-"], input=mlir, capture_output=True, text=True)
    assert p.returncode == 0, p.stderr
    got = RO.evaluate(p.stdout, inputs)
    assert got.dtype == want.dtype and got.shape == want.shape
    assert got.tobytes() == want.tobytes()    # the graph divides the f16 sums the reference wrote
