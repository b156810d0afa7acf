"""CPU oracle for fused-region programs (numpy).  TEST INFRASTRUCTURE ONLY.

Evaluates the text form of a region program -- the thing the generic gfx950
region kernel executes -- with plain numpy: index grids over the iteration
space, fancy indexing for every read, float32 arithmetic, one rounding to the
output type.  Only tests, the smoke check and the benchmark's CPU-baseline leg
may import it; the shipped library never does.

What a program means follows the reference's lowering of fused regions
(paths relative to the reference tree):
  operand maps   Identity / PureBroadcast / PureTranspose / BroadcastTranspose
                 classes, lib/Conversion/LinalgToAscendC/ComputeConversion.cpp:265-333
  body ops       arith.addf / mulf / maximumf (+ subf, divf of the AFIR ops,
                 include/Dialect/AFIR/Ops/Basic/math.td:63-106); relu is
                 maximumf(x, 0), leaky relu is maximumf(x, x*alpha)
                 (examples/matmul-add-leakyrelu/step0_input.mlir:40-52)
  reduction      sum over the last iteration dim, float32 accumulation, output
                 cast (lib/Target/CannKernel/CannTranslation.cpp:2437-2458)
  gather         tensor.extract with one index taken from an index tensor
                 (lib/Conversion/MarkStructuredOps/MarkStructuredOpsPass.cpp:54-147)
  concat         segments writing disjoint row ranges of the output
                 (examples/add-broadcast-concat/step0_input.mlir)
  mean           sum, then operations on the row's sum with constants and extents
                 (examples/broadcast-add-reduce/step0_input_mean.mlir:56-84: sum / N with N
                 an arith.sitofp of the extent).  The IR keeps the sum in an f16 tensor
                 before the division reads it, so the program rounds it there ('reduce sum',
                 'cast f16', then the division in float32 and one rounding to the output type,
                 which for two f16 operands is the correctly rounded f16 quotient).  The
                 reference holds no golden for this graph (its gen_data.py writes the sum
                 only); the test ties the mean to that sum vector
  cast           round to f16 / bf16 (nearest even, overflow to infinity) and widen again:
                 arith.truncf + arith.extf, afir.cast
                 (include/Dialect/AFIR/Ops/Basic/cast.td:22-25), pinned against numpy's
                 float16 conversion and the bf16 bit formula of the comparator
  goldens        "compute in f32, cast to the storage type"
                 (examples/*/gen_data.py, gen_inputs.py)

Pins (tests/test_region_oracle.py): each reference example restated as a
program must reproduce the closed-form golden of that example
(afir_oracle.reduce_rowbias_f16, relu_col_add_f16, relu_colgather_add_f16 and
the concat / split formulas written out with numpy in the test), the five
benchmark configurations as programs must reproduce golden_c1..c4 bit for bit,
single-op programs are checked against Python float arithmetic rounded
through struct, and the graphs of the reference's examples, translated from
MLIR, must turn the reference's own input vectors into its own expected
outputs (tests/golden/reference_examples.npz, tests/test_golden_fixtures.py).  max / min follow IEEE-754 maximum / minimum (-0 < +0, NaN
propagates), which is what arith.maximumf specifies.

Integer regions (_evaluate_integer: afir.add / sub / mul / maximum / minimum /
neg / relu on I16 and I32 tensors, include/Dialect/AFIR/Ops/Basic/math.td:71-98)
are pinned against numpy's own int16 / int32 array arithmetic and against
corner values written out by hand.  Where no intermediate overflows, the result
is fixed by the mathematics.  Where one does, values wrap at the element width,
as numpy (the language of the reference's golden generators) does; the
reference holds no integer golden and lowers these ops to the device's vector
instructions without stating their overflow behaviour, so for overflowing
inputs this function is PARITY UNPINNED.
"""
from __future__ import annotations

import numpy as np

from . import afir_oracle as O

_NP = {"f16": np.float16, "f32": np.float32, "i32": np.int32, "i64": np.int64, "i16": np.int16}


class RegionError(Exception):
    pass


def _ref(tok):
    if tok.startswith("arg"):
        a, d = tok[3:].split(".")
        return ("dim", int(a), int(d))
    return ("const", int(tok))


def parse(text: str) -> dict:
    """Text -> {'args': [(kind, type, rank)], 'segments': [{'rank', 'size',
    'outoff', 'ops': [tuple]}]}."""
    args, segments, seg = [], [], None
    lines = [l.split("#", 1)[0].split() for l in text.splitlines()]
    lines = [l for l in lines if l]
    if not lines or lines[0] != ["afir-hip-region", "1"]:
        raise RegionError("missing header")
    for tok in lines[1:]:
        k = tok[0]
        if k == "arg":
            args.append((tok[1], tok[2], int(tok[3])))
        elif k == "segment":
            seg = {"rank": int(tok[1]), "size": [], "outoff": [("const", 0)], "ops": []}
            segments.append(seg)
        elif k == "end":
            seg = None
        elif k == "size":
            seg["size"] = [_ref(t) for t in tok[1:]]
        elif k == "outoff":
            seg["outoff"] = [_ref(t) for t in tok[1:]]      # terms, summed
        elif k == "push":
            arg = int(tok[1][3:])
            rest = tok[2:]
            sl = []
            if "slice" in rest:
                at = rest.index("slice")
                sl = [_ref(t) for t in rest[at + 1:]]
                rest = rest[:at]
            m = []
            for t in rest:
                if t[0] == "d":
                    m.append(("iter", int(t[1:])))
                elif t[0] == "g":
                    dim, ia = t[1:].split(":")
                    m.append(("gather", int(dim), int(ia[3:])))
                else:
                    m.append(("const", int(t)))
            seg["ops"].append(("push", arg, m, sl))
        elif k == "matmul":
            # 'ta' / 'tb': the operand is stored transposed (linalg.matmul_transpose_a / _b)
            seg["ops"].append(("matmul", int(tok[1][3:]), int(tok[2][3:]), "ta" in tok[3:], "tb" in tok[3:]))
        elif k == "const" and tok[1].startswith("arg"):
            # an extent as a number, rounded through the named float type (f32 when none):
            # arith.sitofp of a cast tensor.dim, examples/broadcast-add-reduce/step0_input_mean.mlir:73-74
            seg["ops"].append(("constref", _ref(tok[1]), tok[2] if len(tok) > 2 else "f32"))
        elif k in ("const", "leaky"):
            seg["ops"].append((k, np.float32(float(tok[1]))))
        elif k == "dup":
            seg["ops"].append(("dup", int(tok[1])))
        elif k == "cast":
            if tok[1] not in ("f16", "bf16", "f32"):
                raise RegionError("cast to a type that is not f16, bf16 or f32")
            seg["ops"].append(("cast", tok[1]))
        elif k == "reduce":
            seg["ops"].append(("reduce",))
        else:
            seg["ops"].append((k,))
    return {"args": args, "segments": segments}


def _widen(arr, t):
    if t == "bf16":
        return O.bf16_bits_to_f32(arr)
    return np.asarray(arr).astype(np.float32)


def ieee_max(a, b):
    r = np.where(a > b, a, np.where(b > a, b, np.where(np.signbit(a), b, a)))
    return np.where(np.isnan(a), a, np.where(np.isnan(b), b, r)).astype(np.float32)


def ieee_min(a, b):
    r = np.where(a < b, a, np.where(b < a, b, np.where(np.signbit(a), a, b)))
    return np.where(np.isnan(a), a, np.where(np.isnan(b), b, r)).astype(np.float32)


def _wrap(v, bits):
    """int64 -> the value `bits`-wide two's complement arithmetic would hold."""
    return ((v + (1 << (bits - 1))) % (1 << bits)) - (1 << (bits - 1))


def _evaluate_integer(prog, inputs, val, out_type, out_rank):
    """Integer regions (afir.add / sub / mul / maximum / minimum / neg / relu on
    I16, I32; include/Dialect/AFIR/Ops/Basic/math.td:71-98): every read is
    converted to the output type and every operation wraps at its width, as a
    graph of afir ops on tensors of that type would."""
    args = prog["args"]
    bits = 16 if out_type == "i16" else 32
    pieces = []
    for seg in prog["segments"]:
        size = [val(r) for r in seg["size"]]
        rank = seg["rank"]
        grids = np.ogrid[tuple(slice(0, s) for s in size)]
        stack = []
        for op in seg["ops"]:
            k = op[0]
            if k == "push":
                _, a, m, sl = op
                if args[a][1] not in ("i16", "i32"):
                    raise RegionError("an integer region reads i16 / i32 tensors only")
                src = np.asarray(inputs[a])
                idx = []
                for d, e in enumerate(m):
                    start = val(sl[d]) if sl else 0
                    if e[0] == "iter":
                        idx.append(grids[e[1]] + start)
                    elif e[0] == "const":
                        idx.append(np.int64(e[1] + start))
                    else:
                        g = np.asarray(inputs[e[2]]).astype(np.int64)[:size[e[1]]]
                        if g.size and (g.min() < 0 or g.max() + start >= src.shape[d]):
                            raise RegionError("gather index out of range")
                        shape = [1] * rank
                        shape[e[1]] = size[e[1]]
                        idx.append(g.reshape(shape) + start)
                v = src[tuple(idx)] if src.ndim else src
                stack.append(_wrap(np.broadcast_to(v, size).astype(np.int64), bits))
            elif k == "const":
                stack.append(_wrap(np.full(size, int(op[1]), dtype=np.int64), bits))
            elif k == "dup":
                stack.append(stack[-1 - op[1]])
            elif k in ("add", "sub", "mul", "max", "min"):
                b, a = stack.pop(), stack.pop()
                stack.append(_wrap({"add": lambda: a + b, "sub": lambda: a - b, "mul": lambda: a * b,
                                      "max": lambda: np.maximum(a, b), "min": lambda: np.minimum(a, b)}[k](), bits))
            elif k == "relu":
                stack.append(np.maximum(stack.pop(), 0))
            elif k == "neg":
                stack.append(_wrap(-stack.pop(), bits))
            elif k == "store":
                pass
            else:
                raise RegionError(f"'{k}' is not available in an integer region")
        if len(stack) != 1:
            raise RegionError("stack does not hold exactly one value at store")
        pieces.append((sum(val(t) for t in seg["outoff"]), stack[0]))
    pieces.sort(key=lambda p: p[0])
    res = np.concatenate([p[1] for p in pieces], axis=0)
    if res.ndim != out_rank:
        raise RegionError("output rank mismatch")
    return res.astype(np.int16 if out_type == "i16" else np.int32)


def evaluate(text: str, inputs, out_shape=None):
    """Runs the program on numpy inputs (bf16 tensors as uint16 bits).  Returns
    the output array in its storage type (bf16 as uint16 bits).  out_shape is
    needed only by programs whose extents refer to the output's dimensions."""
    prog = parse(text)
    args = prog["args"]
    n_in = len(args) - 1
    if len(inputs) != n_in:
        raise RegionError(f"expected {n_in} inputs, got {len(inputs)}")
    shapes = [tuple(x.shape) for x in inputs]
    if out_shape is not None:
        shapes.append(tuple(out_shape))
    out_type, out_rank = args[-1][1], args[-1][2]

    def val(ref):
        return shapes[ref[1]][ref[2]] if ref[0] == "dim" else ref[1]

    if out_type in ("i16", "i32"):
        return _evaluate_integer(prog, inputs, val, out_type, out_rank)

    pieces = []
    for seg in prog["segments"]:
        size = [val(r) for r in seg["size"]]
        rank = seg["rank"]
        grids = np.ogrid[tuple(slice(0, s) for s in size)]
        stack = []
        reduced = False
        for op in seg["ops"]:
            k = op[0]
            if k == "push":
                _, a, m, sl = op
                src = inputs[a]
                idx = []
                for d, e in enumerate(m):
                    start = val(sl[d]) if sl else 0
                    if e[0] == "iter":
                        idx.append(grids[e[1]] + start)
                    elif e[0] == "const":
                        idx.append(np.int64(e[1] + start))
                    else:
                        g = np.asarray(inputs[e[2]]).astype(np.int64)[:size[e[1]]]
                        if g.size and (g.min() < 0 or g.max() + start >= src.shape[d]):
                            raise RegionError("gather index out of range")
                        shape = [1] * rank
                        shape[e[1]] = size[e[1]]
                        idx.append(g.reshape(shape) + start)
                v = _widen(src, args[a][1])[tuple(idx)] if src.ndim else _widen(src, args[a][1])
                stack.append(np.broadcast_to(v, size).astype(np.float32))
            elif k == "matmul":
                # float32 product as the reference golden computes it
                # (examples/matmul-add-leakyrelu/gen_data.py:33: A.f32 @ B.f32)
                # transposed storage is undone first; rank-3 operands are batches of matrices
                # (numpy's @ multiplies the last two dims: linalg.batch_matmul)
                a = _widen(inputs[op[1]], args[op[1]][1])
                b = _widen(inputs[op[2]], args[op[2]][1])
                # (made contiguous: numpy multiplies strided batches without BLAS, 10x slower)
                if op[3]:
                    a = np.ascontiguousarray(np.swapaxes(a, -1, -2))
                if op[4]:
                    b = np.ascontiguousarray(np.swapaxes(b, -1, -2))
                stack.append((a @ b).astype(np.float32))
            elif k == "const":
                stack.append(np.full(size[:-1] if reduced else size, op[1], dtype=np.float32))
            elif k == "constref":
                v = np.float32(val(op[1]))
                if op[2] == "f16":
                    with np.errstate(over="ignore"):
                        v = np.float32(np.float16(v))
                elif op[2] == "bf16":
                    v = O.bf16_bits_to_f32(O.f32_to_bf16_bits(np.array([v], np.float32)))[0]
                stack.append(np.full(size[:-1] if reduced else size, v, dtype=np.float32))
            elif k == "dup":
                stack.append(stack[-1 - op[1]])
            elif k in ("add", "sub", "mul", "div", "max", "min"):
                b, a = stack.pop(), stack.pop()
                with np.errstate(all="ignore"):
                    stack.append({"add": lambda: a + b, "sub": lambda: a - b, "mul": lambda: a * b,
                                  "div": lambda: a / b, "max": lambda: ieee_max(a, b),
                                  "min": lambda: ieee_min(a, b)}[k]().astype(np.float32))
            elif k == "relu":
                stack.append(ieee_max(stack.pop(), np.float32(0)))
            elif k == "leaky":
                x = stack.pop()
                with np.errstate(all="ignore"):
                    stack.append(ieee_max(x, (x * op[1]).astype(np.float32)))
            elif k == "neg":
                stack.append(-stack.pop())
            elif k == "cast":
                # round to the narrower type (nearest even, overflow to infinity) and widen again:
                # arith.truncf followed by arith.extf, afir.cast
                # (include/Dialect/AFIR/Ops/Basic/cast.td:22-25)
                x = stack.pop()
                if op[1] == "f16":
                    with np.errstate(over="ignore"):
                        x = x.astype(np.float16).astype(np.float32)
                elif op[1] == "bf16":
                    x = O.bf16_bits_to_f32(O.f32_to_bf16_bits(np.ascontiguousarray(x, dtype=np.float32))).reshape(x.shape)
                stack.append(x)
            elif k == "reduce":
                # float32 accumulation in numpy's pairwise order, as the
                # reference goldens do it; a kernel's own summation order is
                # compared with a tolerance
                stack.append(np.ascontiguousarray(stack.pop()).sum(axis=-1, dtype=np.float32))
                reduced = True
            elif k == "store":
                pass
            else:
                raise RegionError(f"unknown op {k}")
        if len(stack) != 1:
            raise RegionError("stack does not hold exactly one value at store")
        pieces.append((sum(val(t) for t in seg["outoff"]), stack[0], reduced))
    pieces.sort(key=lambda p: p[0])
    res = np.concatenate([p[1] for p in pieces], axis=0)
    if res.ndim != out_rank:
        raise RegionError("output rank mismatch")
    if out_type == "bf16":
        return O.f32_to_bf16_bits(res.astype(np.float32))
    return res.astype(_NP[out_type])
