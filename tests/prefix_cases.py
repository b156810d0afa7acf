"""Programs that have the form of a hand-tuned family but read only the leading
part of wider tensors (what a zero-offset tensor.extract_slice narrower than
its operand becomes: the extents come from the output or from a constant, the
reads stay plain).  The family kernels assume densely packed operands of exactly
the iteration extents, so such launches must not reach them."""
import numpy as np

from tests.region_cases import HEADER

# out = (a + b) * b on the first 128 columns of [M, 4096] tensors (what the
# translator emits for extract_slice %a[0,0][%m,128] feeding the chain)
ADD_MUL_PREFIX = HEADER + """
arg in f32 2
arg in f32 2
arg out f32 2
segment 2
  size arg0.0 128
  outoff 0
  push arg0 d0 d1
  push arg1 d0 d1
  add
  push arg1 d0 d1
  mul
  store
end
"""

# y[i] = sum_{j < len(bias)} (x[i,j] + bias[j]); x may be wider than bias
ROWSUM_PREFIX = HEADER + """
arg in f32 2
arg in f32 1
arg out f32 1
segment 2
  size arg2.0 arg1.0
  outoff 0
  push arg0 d0 d1
  push arg1 d1
  add
  reduce sum
  store
end
"""

# out[b,j,i] = relu(x[b,i,j]) + c[j] over the extents of out; x may be larger in i and j
TRANSPOSE_PREFIX = HEADER + """
arg in f16 3
arg in f16 1
arg out f16 3
segment 3
  size arg2.0 arg2.1 arg2.2
  outoff 0
  push arg0 d0 d2 d1
  relu
  push arg1 d1
  add
  store
end
"""

# out[r,:] = table[idx[r], :D] * scale + shift with D = out's row length; the table may be wider
GATHER_PREFIX = HEADER + """
arg in f16 2
arg in i32 1
arg in f16 1
arg in f16 1
arg out f16 2
segment 2
  size arg1.0 arg4.1
  outoff 0
  push arg0 g0:arg1 d1
  push arg2 d1
  mul
  push arg3 d1
  add
  store
end
"""


def dims(*shapes):
    return [d for s in shapes for d in s]


# name -> (text, kernel family, shapes that fit the family exactly, shapes that read a prefix)
CASES = {
    "add_mul": (ADD_MUL_PREFIX, "fused_add_mul",
                [(64, 128), (64, 128), (64, 128)], [(64, 4096), (64, 4096), (64, 128)]),
    "add_mul_one_operand": (ADD_MUL_PREFIX, "fused_add_mul",
                            [(64, 128), (64, 128), (64, 128)], [(64, 128), (64, 136), (64, 128)]),
    "rowsum": (ROWSUM_PREFIX, "broadcast_add_reducesum",
               [(96, 4096), (4096,), (96,)], [(96, 8192), (4096,), (96,)]),
    "transpose": (TRANSPOSE_PREFIX, "relu_broadcast_add_transpose",
                  [(3, 128, 64), (64,), (3, 64, 128)], [(3, 192, 64), (64,), (3, 64, 128)]),
    "transpose_cols": (TRANSPOSE_PREFIX, "relu_broadcast_add_transpose",
                       [(3, 128, 64), (64,), (3, 64, 128)], [(3, 128, 72), (72,), (3, 64, 128)]),
    "gather": (GATHER_PREFIX, "gather_scale_shift",
               [(500, 1024), (300,), (1024,), (1024,), (300, 1024)],
               [(500, 2048), (300,), (1024,), (1024,), (300, 1024)]),
}


def make_inputs(text, shapes, seed=3):
    """Seeded inputs for the argument shapes (all but the last, the output)."""
    rng = np.random.default_rng(seed)
    types = [l.split()[2] for l in text.splitlines() if l.split()[:2] == ["arg", "in"]]
    out = []
    for ty, shape in zip(types, shapes[:-1]):
        if ty == "i32":
            out.append(rng.integers(0, shapes[0][0], shape, dtype=np.int64).astype(np.int32))
        else:
            dt = np.float32 if ty == "f32" else np.float16
            out.append(rng.uniform(-1, 1, shape).astype(np.float32).astype(dt))
    return out
