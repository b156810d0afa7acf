"""Region programs used by the CPU and GPU tests: the reference's example
graphs and the benchmark configurations, written in the region-program text
form, each with a seeded input generator and the closed-form golden it must
reproduce (formulas: examples/*/gen_data.py, gen_inputs.py of the reference)."""
import numpy as np

from oracle import afir_oracle as O

HEADER = "afir-hip-region 1\n"


def _u(rng, shape, lo=-1.0, hi=1.0, dt=np.float16):
    return rng.uniform(lo, hi, shape).astype(np.float32).astype(dt)


# c[m] = f16(sum_n (a[m] + b[m,n]))        examples/broadcast-add-reduce
REDUCE_ROWBIAS = HEADER + """
arg in f16 1
arg in f16 2
arg out f16 1
segment 2
  size arg1.0 arg1.1
  outoff 0
  push arg0 d0
  push arg1 d0 d1
  add
  reduce sum
  store
end
"""

# c[m] = f16(sum_n (a[m] + b[m,n]) / N)    examples/broadcast-add-reduce/step0_input_mean.mlir
# (the IR keeps the sums in an f16 tensor before the division reads them: 'cast f16')
MEAN_ROWBIAS = REDUCE_ROWBIAS.replace("  reduce sum\n", "  reduce sum\n  cast f16\n  const arg1.1 f16\n  div\n")
# the sum put through a longer chain: relu(4 - s * 0.5) * (N / 2), extents and constants mixed
REDUCE_TAIL_CHAIN = REDUCE_ROWBIAS.replace(
    "  reduce sum\n", "  reduce sum\n  const 0.5\n  mul\n  neg\n  const 4\n  add\n  relu\n  const arg1.1\n  const 0.5\n  mul\n  mul\n")

# extents outside the tail: out[m,n] = f16(b[m,n] / f16(N) * f32(M)) per element, and a row sum of
# terms that were divided by the extent first, c[m] = f16(sum_n ((a[m] + b[m,n]) / N) * M)
PARALLEL_DIV_EXTENT = HEADER + """
arg in f16 2
arg out f16 2
segment 2
  size arg0.0 arg0.1
  outoff 0
  push arg0 d0 d1
  const arg0.1 f16
  div
  const arg0.0
  mul
  store
end
"""
PRE_REDUCE_DIV_EXTENT = REDUCE_ROWBIAS.replace("  add\n  reduce sum\n", "  add\n  const arg1.1\n  div\n  reduce sum\n  const arg1.0\n  mul\n")

# out[n,m] = f16(relu(data0[m,0]) + data1[n,m])   examples/relu-broadcast-transpose
RELU_COL_ADD = HEADER + """
arg in f16 2
arg in f16 2
arg out f16 2
segment 2
  size arg1.0 arg1.1
  outoff 0
  push arg0 d1 0
  relu
  push arg1 d0 d1
  add
  store
end
"""

# out[i,j] = f16(relu(data[i, idx[j]]) + bias[j])   examples/gather-elementwise-fusion
RELU_COLGATHER_ADD = HEADER + """
arg in f16 2
arg in i64 1
arg in f16 1
arg out f16 2
segment 2
  size arg0.0 arg1.0
  outoff 0
  push arg0 d0 g1:arg1
  relu
  push arg2 d1
  add
  store
end
"""

# rows [0,M): a[m] + b[m,n]; rows [M,2M): c[m] * d[m,n]   examples/add-broadcast-concat
ADD_BROADCAST_CONCAT = HEADER + """
arg in f16 1
arg in f16 2
arg in f16 1
arg in f16 2
arg out f16 2
segment 2
  size arg1.0 arg1.1
  outoff 0
  push arg0 d0
  push arg1 d0 d1
  add
  store
end
segment 2
  size arg3.0 arg3.1
  outoff arg1.0
  push arg2 d0
  push arg3 d0 d1
  mul
  store
end
"""

# halves of a: (relu(a_h) + bias_h[m]) * scale_h[n]        examples/split-relu-brc-add-mul
SPLIT_RELU_BRC_ADD_MUL = HEADER + """
arg in f16 2
arg in f16 1
arg in f16 1
arg in f16 1
arg in f16 1
arg out f16 2
segment 2
  size arg1.0 arg0.1
  outoff 0
  push arg0 d0 d1
  relu
  push arg1 d0
  add
  push arg3 d1
  mul
  store
end
segment 2
  size arg2.0 arg0.1
  outoff arg1.0
  push arg0 d0 d1 slice arg1.0 0
  relu
  push arg2 d0
  add
  push arg4 d1
  mul
  store
end
"""

# the benchmark configurations as programs
C1_ADD_MUL = HEADER + """
arg in f32 2
arg in f32 2
arg out f32 2
segment 2
  size arg0.0 arg0.1
  outoff 0
  push arg0 d0 d1
  push arg1 d0 d1
  add
  push arg1 d0 d1
  mul
  store
end
"""

C2_BCAST_ADD_ROWSUM = HEADER + """
arg in f32 2
arg in f32 1
arg out f32 1
segment 2
  size arg0.0 arg0.1
  outoff 0
  push arg0 d0 d1
  push arg1 d1
  add
  reduce sum
  store
end
"""

# out[b,j,i] = f16(relu(x[b,i,j]) + c[j]): iteration space = output (b, j, i)
C3_RELU_BCAST_TRANSPOSE = HEADER + """
arg in f16 3
arg in f16 1
arg out f16 3
segment 3
  size arg0.0 arg0.2 arg0.1
  outoff 0
  push arg0 d0 d2 d1
  relu
  push arg1 d1
  add
  store
end
"""

C4_GATHER_SCALE_SHIFT = HEADER + """
arg in f16 2
arg in i32 1
arg in f16 1
arg in f16 1
arg out f16 2
segment 2
  size arg1.0 arg0.1
  outoff 0
  push arg0 g0:arg1 d1
  push arg2 d1
  mul
  push arg3 d1
  add
  store
end
"""

# torch_e2e graphs (examples/torch_e2e/test_elementwise.py): (a + b) * c, and an
# AFIR-only chain with sub / div / leaky relu and a dup
ADD_MUL_3 = HEADER + """
arg in f32 2
arg in f32 2
arg in f32 2
arg out f32 2
segment 2
  size arg0.0 arg0.1
  outoff 0
  push arg0 d0 d1
  push arg1 d0 d1
  add
  push arg2 d0 d1
  mul
  store
end
"""

SUB_DIV_LEAKY = HEADER + """
arg in f32 2
arg in f32 1
arg out bf16 2
segment 2
  size arg0.0 arg0.1
  outoff 0
  push arg0 d0 d1
  push arg1 d1
  sub
  dup 0
  const 1.5
  add
  div
  leaky 0.01
  neg
  push arg1 d1
  min
  store
end
"""


def case_reduce_rowbias(m=640, n=512, seed=42):
    rng = np.random.default_rng(seed)
    a, b = _u(rng, (m,)), _u(rng, (m, n))
    return REDUCE_ROWBIAS, [a, b], O.reduce_rowbias_f16(a, b)


def mean_rowbias_f16(a, b):
    """The mean graph's golden: the float32 row sum rounded to f16 (the IR's tensor<?xf16> of
    sums), divided by N (through f16 like the IR's sitofp; exact up to 2048): the correctly
    rounded f16 quotient of two f16 values, computed in float32."""
    n = np.float32(np.float16(b.shape[1]))
    with np.errstate(over="ignore"):
        s = (a.astype(np.float32)[:, None] + b.astype(np.float32)).sum(axis=1, dtype=np.float32).astype(np.float16)
    return (s.astype(np.float32) / n).astype(np.float16)


def case_mean_rowbias(m=640, n=512, seed=42):
    rng = np.random.default_rng(seed)
    a, b = _u(rng, (m,)), _u(rng, (m, n))
    return MEAN_ROWBIAS, [a, b], mean_rowbias_f16(a, b)


def case_parallel_div_extent(m=70, n=333, seed=5):
    rng = np.random.default_rng(seed)
    b = _u(rng, (m, n), -4.0, 4.0)
    want = b.astype(np.float32) / np.float32(np.float16(n)) * np.float32(m)
    return PARALLEL_DIV_EXTENT, [b], want.astype(np.float16)


def case_pre_reduce_div_extent(m=96, n=256, seed=6):
    """Small integers over a power-of-two N: every quotient and every partial sum is exact in
    float32, so the result does not depend on the order of the sum."""
    rng = np.random.default_rng(seed)
    a = rng.integers(-4, 5, (m,)).astype(np.float16)
    b = rng.integers(-4, 5, (m, n)).astype(np.float16)
    terms = (a.astype(np.float32)[:, None] + b.astype(np.float32)) / np.float32(n)
    return PRE_REDUCE_DIV_EXTENT, [a, b], (terms.sum(axis=1, dtype=np.float32) * np.float32(m)).astype(np.float16)


# mixed precision: out = f16((f32(f16(a)) + b) * a), a f32, b f16 per column; and the same
# rounding through bf16 in the middle of a float32 chain, out = f32(bf16(a * b) - b)
CAST_CHAIN_F16 = HEADER + """
arg in f32 2
arg in f16 1
arg out f16 2
segment 2
  size arg0.0 arg0.1
  outoff 0
  push arg0 d0 d1
  cast f16
  push arg1 d1
  add
  push arg0 d0 d1
  mul
  store
end
"""
CAST_CHAIN_BF16 = HEADER + """
arg in f32 2
arg in f32 2
arg out f32 2
segment 2
  size arg0.0 arg0.1
  outoff 0
  push arg0 d0 d1
  push arg1 d0 d1
  mul
  cast bf16
  push arg1 d0 d1
  sub
  store
end
"""


def _special_f32(rng, shape):
    """Uniform values with the float32 corner cases of a rounding mixed in: ties, values that
    overflow f16, f16 subnormals, infinities, NaN, both zeros."""
    x = rng.uniform(-4, 4, shape).astype(np.float32)
    flat = x.reshape(-1)
    corners = np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e6, -1e6, 6e-8, 3e-8, 2.98e-8, np.inf, -np.inf, np.nan,
                        1.0 + 2.0 ** -11, 1.0 + 3 * 2.0 ** -11, 2049.0, 2051.0, 1.0 + 2.0 ** -8, 1.0 + 3 * 2.0 ** -8],
                       np.float32)
    flat[:corners.size] = corners
    return x


def case_cast_chain_f16(m=70, n=333, seed=11):
    rng = np.random.default_rng(seed)
    a = _special_f32(rng, (m, n))
    b = rng.uniform(-2, 2, (n,)).astype(np.float16)
    with np.errstate(all="ignore"):
        want = ((a.astype(np.float16).astype(np.float32) + b.astype(np.float32)) * a).astype(np.float16)
    return CAST_CHAIN_F16, [a, b], want


def case_cast_chain_bf16(m=64, n=256, seed=12):
    rng = np.random.default_rng(seed)
    a = _special_f32(rng, (m, n))
    b = rng.uniform(-2, 2, (m, n)).astype(np.float32)
    with np.errstate(all="ignore"):
        p = (a * b).astype(np.float32)
        rounded = O.bf16_bits_to_f32(O.f32_to_bf16_bits(p))
        want = (rounded - b).astype(np.float32)
    return CAST_CHAIN_BF16, [a, b], want


def case_reduce_tail_chain(m=77, n=300, seed=9):
    rng = np.random.default_rng(seed)
    a, b = _u(rng, (m,)), _u(rng, (m, n), -0.1, 0.1)
    s = (a.astype(np.float32)[:, None] + b.astype(np.float32)).sum(axis=1, dtype=np.float32)
    t = np.maximum(np.float32(4) + -(s * np.float32(0.5)), np.float32(0))
    return REDUCE_TAIL_CHAIN, [a, b], (t * (np.float32(n) * np.float32(0.5))).astype(np.float16)


def case_relu_col_add(m=640, n=500, seed=42):
    rng = np.random.default_rng(seed)
    d0, d1 = _u(rng, (m, 1)), _u(rng, (n, m))
    return RELU_COL_ADD, [d0, d1], O.relu_col_add_f16(d0, d1)


def case_relu_colgather_add(m=16, n=640, k=128, seed=42):
    rng = np.random.default_rng(seed)
    data, bias = _u(rng, (m, n)), _u(rng, (k,))
    idx = rng.integers(0, n, k, dtype=np.int64)
    return RELU_COLGATHER_ADD, [data, idx, bias], O.relu_colgather_add_f16(data, idx, bias)


def case_add_broadcast_concat(m=320, n=512, seed=42):
    rng = np.random.default_rng(seed)
    a, b, c, d = _u(rng, (m,)), _u(rng, (m, n)), _u(rng, (m,)), _u(rng, (m, n))
    want = np.concatenate([(a[:, None].astype(np.float32) + b.astype(np.float32)),
                           (c[:, None].astype(np.float32) * d.astype(np.float32))],
                          axis=0).astype(np.float16)
    return ADD_BROADCAST_CONCAT, [a, b, c, d], want


def case_split_relu_brc_add_mul(m=640, n=512, seed=42):
    rng = np.random.default_rng(seed)
    hm = m // 2
    a = _u(rng, (m, n))
    b0, b1, s0, s1 = _u(rng, (hm,)), _u(rng, (hm,)), _u(rng, (n,)), _u(rng, (n,))
    f = np.float32
    o0 = (np.maximum(a[:hm].astype(f), f(0)) + b0[:, None].astype(f)) * s0[None, :].astype(f)
    o1 = (np.maximum(a[hm:].astype(f), f(0)) + b1[:, None].astype(f)) * s1[None, :].astype(f)
    return SPLIT_RELU_BRC_ADD_MUL, [a, b0, b1, s0, s1], np.concatenate([o0, o1], 0).astype(np.float16)


def case_c1(shape=(96, 1000)):
    a, b = O.gen_c1(shape)
    return C1_ADD_MUL, [a, b], O.golden_c1(a, b)


def case_c2(m=64, n=4096):
    x, bias = O.gen_c2(m, n)
    return C2_BCAST_ADD_ROWSUM, [x, bias], O.golden_c2(x, bias)


def case_c3(b=2, m=96, n=64):
    x, c = O.gen_c3(b, m, n)
    return C3_RELU_BCAST_TRANSPOSE, [x, c], O.golden_c3(x, c)


def case_c4(rows=512, dim=264, nidx=300):
    table, idx, scale, shift = O.gen_c4(rows, dim, nidx)
    return C4_GATHER_SCALE_SHIFT, [table, idx, scale, shift], O.golden_c4(table, idx, scale, shift)


def case_add_mul_3(shape=(33, 77), seed=5):
    rng = np.random.default_rng(seed)
    a, b, c = (_u(rng, shape, dt=np.float32) for _ in range(3))
    return ADD_MUL_3, [a, b, c], ((a + b) * c).astype(np.float32)


EXACT_CASES = {
    "relu_col_add": case_relu_col_add,
    "relu_colgather_add": case_relu_colgather_add,
    "add_broadcast_concat": case_add_broadcast_concat,
    "split_relu_brc_add_mul": case_split_relu_brc_add_mul,
    "c1": case_c1, "c3": case_c3, "c4": case_c4, "add_mul_3": case_add_mul_3,
    "parallel_div_extent": case_parallel_div_extent, "pre_reduce_div_extent": case_pre_reduce_div_extent,
    "cast_chain_f16": case_cast_chain_f16, "cast_chain_bf16": case_cast_chain_bf16,
}
REDUCE_CASES = {"reduce_rowbias": case_reduce_rowbias, "c2": case_c2, "mean_rowbias": case_mean_rowbias,
                "reduce_tail_chain": case_reduce_tail_chain}


# Hand-written static kernels of the reference's multi-kernel examples
# (examples/real-npu-microcases/kernels/const640.cpp: every element 1,
# const_with_input640.cpp: every element 2, its input ignored,
# copy_scalar640.cpp: a copy; examples/real-npu-multikernel/kernels/add_wait640.cpp:
# lhs + rhs), as region programs.
CONST_ONE = HEADER + "arg out f16 1\nsegment 1\n size arg0.0\n outoff 0\n const 1\n store\nend\n"
CONST_TWO_IGNORING_INPUT = HEADER + "arg in f16 1\narg out f16 1\nsegment 1\n size arg1.0\n outoff 0\n const 2\n store\nend\n"
COPY_1D = HEADER + "arg in f16 1\narg out f16 1\nsegment 1\n size arg1.0\n outoff 0\n push arg0 d0\n store\nend\n"
ADD_1D = (HEADER + "arg in f16 1\narg in f16 1\narg out f16 1\nsegment 1\n size arg2.0\n outoff 0\n"
          " push arg0 d0\n push arg1 d0\n add\n store\nend\n")


# Integer regions: afir.add / sub / mul / maximum / minimum / neg / relu on I16 and
# I32 tensors (include/Dialect/AFIR/Ops/Basic/math.td:71-98; the reference's
# convert_add_i32 and test_add_i16 functions, test/Conversion/afir_to_ascir.mlir:34-37,
# test/Dialect/AFIR/ops.mlir:8-11).  Expected values come from numpy's own fixed
# width integer arithmetic, which wraps like the kernels' 32-bit registers.
INT_ADD_I32 = (HEADER + "arg in i32 2\narg in i32 2\narg out i32 2\nsegment 2\n size arg0.0 arg0.1\n outoff 0\n"
               " push arg0 d0 d1\n push arg1 d0 d1\n add\n store\nend\n")
INT_ADD_I16 = INT_ADD_I32.replace("i32", "i16")
# relu(x - row) * col + min(x, -x), the transposed read included
INT_CHAIN_I32 = HEADER + """
arg in i32 2
arg in i32 1
arg in i32 1
arg in i32 2
arg out i32 2
segment 2
  size arg0.0 arg0.1
  outoff 0
  push arg0 d0 d1
  push arg1 d0
  sub
  relu
  push arg2 d1
  mul
  push arg0 d0 d1
  dup 0
  neg
  min
  add
  push arg3 d1 d0
  max
  const -7
  add
  store
end
"""
# the same on i16 tensors: comparisons see values wrapped to 16 bits
INT_CHAIN_I16 = INT_CHAIN_I32.replace("i32", "i16")
# i16 and i32 reads in one region, i16 result (every value taken modulo 2^16)
INT_MIXED_TO_I16 = HEADER + """
arg in i16 2
arg in i32 1
arg out i16 2
segment 2
  size arg0.0 arg0.1
  outoff 0
  push arg0 d0 d1
  push arg1 d1
  mul
  push arg0 d0 d1
  add
  store
end
"""
# rows of an i32 table picked by an index tensor, plus a per-column i16 term
INT_GATHER_ROWS = HEADER + """
arg in i32 2
arg in i64 1
arg in i16 1
arg out i32 2
segment 2
  size arg1.0 arg0.1
  outoff 0
  push arg0 g0:arg1 d1
  push arg2 d1
  add
  store
end
"""


def _ints(rng, shape, dt):
    """Full-range values with the overflow-prone ones seeded in."""
    info = np.iinfo(dt)
    x = rng.integers(info.min, info.max, shape, dtype=dt, endpoint=True)
    flat = x.reshape(-1)
    special = np.array([info.min, info.max, 0, -1, 1, info.min + 1], dtype=dt)
    if flat.size:
        where = rng.integers(0, flat.size, min(flat.size, 12))
        flat[where] = special[np.arange(where.size) % special.size]
    return x


def case_int_add_i32(shape=(37, 203), seed=11):
    rng = np.random.default_rng(seed)
    a, b = _ints(rng, shape, np.int32), _ints(rng, shape, np.int32)
    with np.errstate(over="ignore"):
        return INT_ADD_I32, [a, b], a + b


def case_int_add_i16(shape=(37, 203), seed=12):
    rng = np.random.default_rng(seed)
    a, b = _ints(rng, shape, np.int16), _ints(rng, shape, np.int16)
    with np.errstate(over="ignore"):
        return INT_ADD_I16, [a, b], a + b


def case_int_chain_i32(m=70, n=130, seed=13, dt=np.int32, text=INT_CHAIN_I32):
    rng = np.random.default_rng(seed)
    x, r, c, t = _ints(rng, (m, n), dt), _ints(rng, (m,), dt), _ints(rng, (n,), dt), _ints(rng, (n, m), dt)
    with np.errstate(over="ignore"):
        v = np.maximum(x - r[:, None], dt(0)) * c[None, :]
        v = v + np.minimum(x, -x)
        v = np.maximum(v, t.T) + dt(-7)
    assert v.dtype == dt
    return text, [x, r, c, t], v


def case_int_chain_i16(m=70, n=130, seed=16):
    return case_int_chain_i32(m, n, seed, np.int16, INT_CHAIN_I16)


def case_int_mixed_to_i16(m=33, n=77, seed=14):
    rng = np.random.default_rng(seed)
    x, c = _ints(rng, (m, n), np.int16), _ints(rng, (n,), np.int32)
    with np.errstate(over="ignore"):
        v = x * c.astype(np.int16)[None, :] + x            # numpy's narrowing cast keeps the low 16 bits
    return INT_MIXED_TO_I16, [x, c], v


def case_int_gather_rows(rows=300, n=96, nidx=45, seed=15):
    rng = np.random.default_rng(seed)
    table, col = _ints(rng, (rows, n), np.int32), _ints(rng, (n,), np.int16)
    idx = rng.integers(0, rows, (nidx,), dtype=np.int64)
    with np.errstate(over="ignore"):
        return INT_GATHER_ROWS, [table, idx, col], table[idx] + col.astype(np.int32)[None, :]


INT_CASES = {
    "int_add_i32": case_int_add_i32, "int_add_i16": case_int_add_i16, "int_chain_i32": case_int_chain_i32,
    "int_chain_i16": case_int_chain_i16,
    "int_mixed_to_i16": case_int_mixed_to_i16, "int_gather_rows": case_int_gather_rows,
}
