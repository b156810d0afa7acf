"""The reference's own vectors (tests/golden/reference_examples.npz, written by
tests/golden/make_fixtures.py from the reference's golden scripts) paired with
the MLIR graph / region program that computes each of them."""
import os

import numpy as np

from tests import mlir_cases as MC
from tests import region_cases as RC

FIXTURE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_examples.npz")

RELU_ONLY = RC.HEADER + "arg in f16 1\narg out f16 1\nsegment 1\n size arg0.0\n outoff 0\n push arg0 d0\n relu\n store\nend\n"
# expected[i, j] = base[0, j] + bias[i, j]   (examples/real-npu-microcases/gen_data.py:99-106)
BROADCAST_ADD = RC.HEADER + ("arg in f16 2\narg in f16 2\narg out f16 2\nsegment 2\n size arg1.0 arg1.1\n outoff 0\n"
                             " push arg0 0 d1\n push arg1 d0 d1\n add\n store\nend\n")


def load():
    return np.load(FIXTURE, allow_pickle=False)


def cases():
    """name -> (mlir text or None, region program or None, inputs, expected, exact)"""
    z = load()
    g = lambda k: np.ascontiguousarray(z[k])
    e = "broadcast-add-reduce/"
    yield "broadcast-add-reduce", MC.ROW_BIAS_REDUCE, None, [g(e + "input_a"), g(e + "input_b")], g(e + "output_c"), False
    e = "relu-broadcast-transpose/"
    yield ("relu-broadcast-transpose", MC.RELU_COLUMN_ADD, None,
           [g(e + "input_data0"), g(e + "input_data1")], g(e + "output_expected"), True)
    e = "gather-elementwise-fusion/"
    yield ("gather-elementwise-fusion", MC.RELU_GATHER_COLUMNS_ADD, None,
           [g(e + "input_data"), g(e + "input_indices"), g(e + "input_bias")], g(e + "output_out"), True)
    e = "matmul-add-leakyrelu/"
    out = g(e + "output")
    yield ("matmul-add-leakyrelu", MC.MATMUL_BIAS_LEAKY_F16, None,
           [g(e + "input_a"), g(e + "input_b"), g(e + "input_bias"), np.zeros_like(out)], out, True)
    e = "add-broadcast-concat/"
    yield ("add-broadcast-concat", MC.TWO_CHAINS_CONCAT, None,
           [g(e + "input_a"), g(e + "input_b"), g(e + "input_c"), g(e + "input_d")], g(e + "output"), True)
    e = "split-relu-brc-add-mul/"
    yield ("split-relu-brc-add-mul", MC.SPLIT_HALVES, None,
           [g(e + "input_a"), g(e + "bias0"), g(e + "bias1"), g(e + "scale0"), g(e + "scale1")], g(e + "output"), True)
    e = "real-npu-microcases/relu_only/"
    yield "microcase-relu_only", None, RELU_ONLY, [g(e + "input")], g(e + "expected"), True
    e = "real-npu-microcases/broadcast_add/"
    yield "microcase-broadcast_add", None, BROADCAST_ADD, [g(e + "input"), g(e + "bias")], g(e + "expected"), True


def mean_case():
    """The reference's mean graph (examples/broadcast-add-reduce/step0_input_mean.mlir) on the vectors its
    gen_data.py wrote for the sum.  The reference holds no mean output, but output_c is the f16 tensor of
    sums that the graph's division reads: mean = output_c / N, rounded once."""
    z = load()
    e = "broadcast-add-reduce/"
    a, b, c = (np.ascontiguousarray(z[e + k]) for k in ("input_a", "input_b", "output_c"))
    want = (c.astype(np.float32) / np.float32(b.shape[1])).astype(np.float16)
    return MC.ROW_BIAS_MEAN, [a, b], want


def within_one_f16_ulp(got, want):
    g = got.astype(np.float64)
    w = want.astype(np.float64)
    ulp = np.maximum(np.abs(np.spacing(want).astype(np.float64)), 2.0 ** -24)
    return bool(np.all(np.abs(g - w) <= ulp))
