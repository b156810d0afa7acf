"""MLIR inputs for the translator tests, written in the syntax of the
reference's example graphs (examples/*/step0_input.mlir) and AFIR tests
(test/Dialect/AFIR/ops.mlir, README.md:191-197): same op vocabulary and
structure, this repository's own text."""

ROW_BIAS_REDUCE = """
// c[m] = sum_n (a[m] + b[m, n])
#row = affine_map<(d0, d1) -> (d0)>
#all = affine_map<(d0, d1) -> (d0, d1)>
module {
  func.func @rowbias_reduce(%a : tensor<?xf16>, %b : tensor<?x?xf16>) -> tensor<?xf16> {
    %c0 = arith.constant 0 : index
    %c1 = arith.constant 1 : index
    %m = tensor.dim %a, %c0 : tensor<?xf16>
    %n = tensor.dim %b, %c1 : tensor<?x?xf16>
    %e0 = tensor.empty(%m, %n) : tensor<?x?xf16>
    %bc = linalg.generic {indexing_maps = [#row, #all], iterator_types = ["parallel", "parallel"]}
        ins(%a : tensor<?xf16>) outs(%e0 : tensor<?x?xf16>) {
      ^bb0(%x: f16, %o: f16):
        linalg.yield %x : f16
    } -> tensor<?x?xf16>
    %e1 = tensor.empty(%m, %n) : tensor<?x?xf16>
    %sum = linalg.generic {indexing_maps = [#all, #all, #all], iterator_types = ["parallel", "parallel"]}
        ins(%bc, %b : tensor<?x?xf16>, tensor<?x?xf16>) outs(%e1 : tensor<?x?xf16>) {
      ^bb0(%x: f16, %y: f16, %o: f16):
        %s = arith.addf %x, %y : f16
        linalg.yield %s : f16
    } -> tensor<?x?xf16>
    %zero = arith.constant 0.0 : f16
    %e2 = tensor.empty(%m) : tensor<?xf16>
    %init = linalg.fill ins(%zero : f16) outs(%e2 : tensor<?xf16>) -> tensor<?xf16>
    %red = linalg.generic {indexing_maps = [#all, #row], iterator_types = ["parallel", "reduction"]}
        ins(%sum : tensor<?x?xf16>) outs(%init : tensor<?xf16>) {
      ^bb0(%x: f16, %acc: f16):
        %s = arith.addf %acc, %x : f16
        linalg.yield %s : f16
    } -> tensor<?xf16>
    return %red : tensor<?xf16>
  }
}
"""

# the same graph followed by a division by N: the reference's mean example
# (examples/broadcast-add-reduce/step0_input_mean.mlir:56-84), N as arith.sitofp of the extent
ROW_BIAS_MEAN = ROW_BIAS_REDUCE.replace("@rowbias_reduce", "@rowbias_mean").replace(
    "    return %red : tensor<?xf16>\n", """    %ni = arith.index_cast %n : index to i32
    %nf = arith.sitofp %ni : i32 to f16
    %e3 = tensor.empty(%m) : tensor<?xf16>
    %mean = linalg.generic {indexing_maps = [#row1, #row1], iterator_types = ["parallel"]}
        ins(%red : tensor<?xf16>) outs(%e3 : tensor<?xf16>) {
      ^bb0(%x: f16, %o: f16):
        %q = arith.divf %x, %nf : f16
        linalg.yield %q : f16
    } -> tensor<?xf16>
    return %mean : tensor<?xf16>
""").replace("#all = affine_map", "#row1 = affine_map<(d0) -> (d0)>\n#all = affine_map")

RELU_COLUMN_ADD = """
// out[n, m] = relu(col[m, 0]) + d[n, m]
func.func @relu_column_add(%col: tensor<?x1xf16>, %d: tensor<?x?xf16>) -> tensor<?x?xf16> {
  %c0 = arith.constant 0 : index
  %m = tensor.dim %col, %c0 : tensor<?x1xf16>
  %n = tensor.dim %d, %c0 : tensor<?x?xf16>
  %z = arith.constant 0.0 : f16
  %e0 = tensor.empty(%m) : tensor<?x1xf16>
  %r = linalg.generic {
      indexing_maps = [affine_map<(d0, d1) -> (d0, d1)>, affine_map<(d0, d1) -> (d0, d1)>],
      iterator_types = ["parallel", "parallel"]
    } ins(%col : tensor<?x1xf16>) outs(%e0 : tensor<?x1xf16>) {
    ^bb0(%x: f16, %o: f16):
      %v = arith.maximumf %x, %z : f16
      linalg.yield %v : f16
  } -> tensor<?x1xf16>
  %e1 = tensor.empty(%n, %m) : tensor<?x?xf16>
  %res = linalg.generic {
      indexing_maps = [affine_map<(d0, d1) -> (d1, 0)>, affine_map<(d0, d1) -> (d0, d1)>,
                       affine_map<(d0, d1) -> (d0, d1)>],
      iterator_types = ["parallel", "parallel"]
    } ins(%r, %d : tensor<?x1xf16>, tensor<?x?xf16>) outs(%e1 : tensor<?x?xf16>) {
    ^bb0(%x: f16, %y: f16, %o: f16):
      %s = arith.addf %x, %y : f16
      linalg.yield %s : f16
  } -> tensor<?x?xf16>
  return %res : tensor<?x?xf16>
}
"""

RELU_GATHER_COLUMNS_ADD = """
// out[i, j] = relu(data[i, idx[j]]) + bias[j]
#col = affine_map<(d0, d1) -> (d1)>
#all = affine_map<(d0, d1) -> (d0, d1)>
func.func @relu_gather_columns_add(%data : tensor<?x?xf16>, %idx : tensor<?xi64>, %bias : tensor<?xf16>)
    -> tensor<?x?xf16> {
  %c0 = arith.constant 0 : index
  %c1 = arith.constant 1 : index
  %z = arith.constant 0.0 : f16
  %m = tensor.dim %data, %c0 : tensor<?x?xf16>
  %n = tensor.dim %data, %c1 : tensor<?x?xf16>
  %k = tensor.dim %idx, %c0 : tensor<?xi64>
  %e0 = tensor.empty(%m, %n) : tensor<?x?xf16>
  %r = linalg.generic {indexing_maps = [#all, #all], iterator_types = ["parallel", "parallel"]}
      ins(%data : tensor<?x?xf16>) outs(%e0 : tensor<?x?xf16>) {
    ^bb0(%x: f16, %o: f16):
      %v = arith.maximumf %x, %z : f16
      linalg.yield %v : f16
  } -> tensor<?x?xf16>
  %e1 = tensor.empty(%m, %k) : tensor<?x?xf16>
  %g = linalg.generic {indexing_maps = [#col, #all], iterator_types = ["parallel", "parallel"]}
      ins(%idx : tensor<?xi64>) outs(%e1 : tensor<?x?xf16>) {
    ^bb0(%ix: i64, %o: f16):
      %i = linalg.index 0 : index
      %p = arith.index_cast %ix : i64 to index
      %v = tensor.extract %r[%i, %p] : tensor<?x?xf16>
      linalg.yield %v : f16
  } -> tensor<?x?xf16>
  %e2 = tensor.empty(%m, %k) : tensor<?x?xf16>
  %res = linalg.generic {indexing_maps = [#all, #col, #all], iterator_types = ["parallel", "parallel"]}
      ins(%g, %bias : tensor<?x?xf16>, tensor<?xf16>) outs(%e2 : tensor<?x?xf16>) {
    ^bb0(%x: f16, %b: f16, %o: f16):
      %s = arith.addf %x, %b : f16
      linalg.yield %s : f16
  } -> tensor<?x?xf16>
  return %res : tensor<?x?xf16>
}
"""

MATMUL_BIAS_LEAKY_F16 = """
#bias = affine_map<(d0, d1) -> (d1)>
#all = affine_map<(d0, d1) -> (d0, d1)>
func.func @mm_bias_leaky(%a : tensor<?x?xf16>, %b : tensor<?x?xf16>, %bias : tensor<?xf32>,
                         %init : tensor<?x?xf32>) -> tensor<?x?xf32> {
  %c0 = arith.constant 0 : index
  %c1 = arith.constant 1 : index
  %m = tensor.dim %init, %c0 : tensor<?x?xf32>
  %n = tensor.dim %init, %c1 : tensor<?x?xf32>
  %c = linalg.matmul ins(%a, %b : tensor<?x?xf16>, tensor<?x?xf16>) outs(%init : tensor<?x?xf32>) -> tensor<?x?xf32>
  %e0 = tensor.empty(%m, %n) : tensor<?x?xf32>
  %d = linalg.generic {indexing_maps = [#all, #bias, #all], iterator_types = ["parallel", "parallel"]}
      ins(%c, %bias : tensor<?x?xf32>, tensor<?xf32>) outs(%e0 : tensor<?x?xf32>) {
    ^bb0(%x: f32, %y: f32, %o: f32):
      %s = arith.addf %x, %y : f32
      linalg.yield %s : f32
  } -> tensor<?x?xf32>
  %alpha = arith.constant 1.0e-3 : f32
  %e1 = tensor.empty(%m, %n) : tensor<?x?xf32>
  %e = linalg.generic {indexing_maps = [#all, #all], iterator_types = ["parallel", "parallel"]}
      ins(%d : tensor<?x?xf32>) outs(%e1 : tensor<?x?xf32>) {
    ^bb0(%x: f32, %o: f32):
      %t = arith.mulf %x, %alpha : f32
      %v = arith.maximumf %x, %t : f32
      linalg.yield %v : f32
  } -> tensor<?x?xf32>
  return %e : tensor<?x?xf32>
}
"""

MATMUL_BIAS_LEAKY_BF16 = MATMUL_BIAS_LEAKY_F16.replace("xf16", "xbf16").replace("f32", "bf16") \
    .replace("1.0e-3", "1.0e-2").replace("@mm_bias_leaky", "@mm_bias_leaky_bf16")

# The other epilogue kinds the reference's matmul annotation knows
# (test/Conversion/annotate-mix-matmul-semantics.mlir:3-25: "None", "BiasAdd").
MATMUL_PLAIN_F16 = """
func.func @mm_plain(%a : tensor<?x?xf16>, %b : tensor<?x?xf16>, %init : tensor<?x?xf32>) -> tensor<?x?xf32> {
  %c = linalg.matmul ins(%a, %b : tensor<?x?xf16>, tensor<?x?xf16>) outs(%init : tensor<?x?xf32>) -> tensor<?x?xf32>
  return %c : tensor<?x?xf32>
}
"""

MATMUL_BIAS_F16 = """
#bias = affine_map<(d0, d1) -> (d1)>
#all = affine_map<(d0, d1) -> (d0, d1)>
func.func @mm_bias(%a : tensor<?x?xf16>, %b : tensor<?x?xf16>, %bias : tensor<?xf32>,
                   %init : tensor<?x?xf32>) -> tensor<?x?xf32> {
  %c0 = arith.constant 0 : index
  %c1 = arith.constant 1 : index
  %m = tensor.dim %init, %c0 : tensor<?x?xf32>
  %n = tensor.dim %init, %c1 : tensor<?x?xf32>
  %c = linalg.matmul ins(%a, %b : tensor<?x?xf16>, tensor<?x?xf16>) outs(%init : tensor<?x?xf32>) -> tensor<?x?xf32>
  %e0 = tensor.empty(%m, %n) : tensor<?x?xf32>
  %d = linalg.generic {indexing_maps = [#all, #bias, #all], iterator_types = ["parallel", "parallel"]}
      ins(%c, %bias : tensor<?x?xf32>, tensor<?xf32>) outs(%e0 : tensor<?x?xf32>) {
    ^bb0(%x: f32, %y: f32, %o: f32):
      %s = arith.addf %x, %y : f32
      linalg.yield %s : f32
  } -> tensor<?x?xf32>
  return %d : tensor<?x?xf32>
}
"""
MATMUL_PLAIN_BF16 = MATMUL_PLAIN_F16.replace("xf16", "xbf16").replace("f32", "bf16").replace("@mm_plain", "@mm_plain_bf16")
MATMUL_BIAS_BF16 = MATMUL_BIAS_F16.replace("xf16", "xbf16").replace("f32", "bf16").replace("@mm_bias", "@mm_bias_bf16")

# matmul -> bias add -> relu, and matmul -> relu: the runtime's BiasAddRelu epilogue
# (include/Runtime/Mix/MatmulTilingTypes.h:13); relu spelled maximumf(x, 0.0) as in
# test/Target/cann-translate-mix-relu-input.mlir.
MATMUL_BIAS_RELU_F16 = MATMUL_BIAS_LEAKY_F16.replace("%alpha = arith.constant 1.0e-3 : f32", "%alpha = arith.constant 0.0 : f32") \
    .replace("      %t = arith.mulf %x, %alpha : f32\n", "").replace("arith.maximumf %x, %t", "arith.maximumf %x, %alpha") \
    .replace("@mm_bias_leaky", "@mm_bias_relu")
MATMUL_BIAS_RELU_BF16 = MATMUL_BIAS_RELU_F16.replace("xf16", "xbf16").replace("f32", "bf16").replace("@mm_bias_relu", "@mm_bias_relu_bf16")
MATMUL_RELU_F16 = """
#all = affine_map<(d0, d1) -> (d0, d1)>
func.func @mm_relu(%a : tensor<?x?xf16>, %b : tensor<?x?xf16>, %init : tensor<?x?xf32>) -> tensor<?x?xf32> {
  %c0 = arith.constant 0 : index
  %c1 = arith.constant 1 : index
  %m = tensor.dim %init, %c0 : tensor<?x?xf32>
  %n = tensor.dim %init, %c1 : tensor<?x?xf32>
  %c = linalg.matmul ins(%a, %b : tensor<?x?xf16>, tensor<?x?xf16>) outs(%init : tensor<?x?xf32>) -> tensor<?x?xf32>
  %zero = arith.constant 0.0 : f32
  %e1 = tensor.empty(%m, %n) : tensor<?x?xf32>
  %e = linalg.generic {indexing_maps = [#all, #all], iterator_types = ["parallel", "parallel"]}
      ins(%c : tensor<?x?xf32>) outs(%e1 : tensor<?x?xf32>) {
    ^bb0(%x: f32, %o: f32):
      %v = arith.maximumf %x, %zero : f32
      linalg.yield %v : f32
  } -> tensor<?x?xf32>
  return %e : tensor<?x?xf32>
}
"""
MATMUL_RELU_BF16 = MATMUL_RELU_F16.replace("xf16", "xbf16").replace("f32", "bf16").replace("@mm_relu", "@mm_relu_bf16")

# An AscGraph in AFIR form (the structure of python/afir-to-ascir/asc_graph.afir:1-13:
# load, load, broadcast, add, mul, sub, store, every op with an attribute
# dictionary): out = (x + y) - (x + y) * y with y broadcast over the rows.
ASC_GRAPH_FORM = """
#id = affine_map<(d0, d1) -> (d0, d1)>
module attributes {afir.asc_graph_attr = #afir.asc_graph<axes = [<id = 0, name = "r", axis_type = Original, size = "12">, <id = 1, name = "c", axis_type = Original, size = "40">], type = Compute>} {
  func.func @asc_graph(%x: tensor<12x40xf32>, %y: tensor<1x40xf32>) -> tensor<12x40xf32> {
    %lx = afir.load %x {indexing_maps = [#id], ir_attr_def = {offset = "0"}, outputs = [#afir.asc_tensor<tensor_id = -1, position = <gm>>]} : tensor<12x40xf32> -> tensor<12x40xf32>
    %ly = afir.load %y {indexing_maps = [#id], ir_attr_def = {offset = "0"}, outputs = [#afir.asc_tensor<tensor_id = -1, position = <gm>>]} : tensor<1x40xf32> -> tensor<1x40xf32>
    %by = afir.broadcast %ly {indexing_maps = [#id], outputs = [#afir.asc_tensor<tensor_id = -1, position = <gm>>]} : tensor<1x40xf32> -> tensor<12x40xf32>
    %s = afir.add %lx, %by {indexing_maps = [#id, #id, #id], outputs = [#afir.asc_tensor<tensor_id = -1, position = <gm>>]} : (tensor<12x40xf32>, tensor<12x40xf32>) -> tensor<12x40xf32>
    %p = afir.mul %s, %by {indexing_maps = [#id, #id, #id], outputs = [#afir.asc_tensor<tensor_id = -1, position = <gm>>]} : (tensor<12x40xf32>, tensor<12x40xf32>) -> tensor<12x40xf32>
    %d = afir.sub %s, %p {indexing_maps = [#id, #id, #id], outputs = [#afir.asc_tensor<tensor_id = -1, position = <gm>>]} : (tensor<12x40xf32>, tensor<12x40xf32>) -> tensor<12x40xf32>
    %o = afir.store %d {indexing_maps = [#id], outputs = [#afir.asc_tensor<tensor_id = -1, position = <gm>>]} : tensor<12x40xf32> -> tensor<12x40xf32>
    return %o : tensor<12x40xf32>
  }
}
"""

# afir.concat of three parts along axis 0 (the op form of
# test/Dialect/AFIR/ops.mlir:350-355), each part an elementwise value.
THREE_PART_CONCAT = """
func.func @concat3(%a: tensor<?x?xf32>, %b: tensor<?x?xf32>, %c: tensor<?x?xf32>) -> tensor<?x?xf32> {
  %ra = afir.relu %a : tensor<?x?xf32> -> tensor<?x?xf32>
  %nb = afir.neg %b : tensor<?x?xf32> -> tensor<?x?xf32>
  %0 = afir.concat %ra, %nb, %c {concat_axis = 0 : i32} : tensor<?x?xf32>, tensor<?x?xf32>, tensor<?x?xf32> -> tensor<?x?xf32>
  return %0 : tensor<?x?xf32>
}
"""

TWO_CHAINS_CONCAT = """
#row = affine_map<(d0, d1) -> (d0)>
#all = affine_map<(d0, d1) -> (d0, d1)>
func.func @two_chains_concat(%a : tensor<?xf16>, %b : tensor<?x?xf16>, %c : tensor<?xf16>,
                             %d : tensor<?x?xf16>) -> tensor<?x?xf16> {
  %c0 = arith.constant 0 : index
  %c1 = arith.constant 1 : index
  %m = tensor.dim %a, %c0 : tensor<?xf16>
  %n = tensor.dim %b, %c1 : tensor<?x?xf16>
  %e0 = tensor.empty(%m, %n) : tensor<?x?xf16>
  %s = linalg.generic {indexing_maps = [#row, #all, #all], iterator_types = ["parallel", "parallel"]}
      ins(%a, %b : tensor<?xf16>, tensor<?x?xf16>) outs(%e0 : tensor<?x?xf16>) {
    ^bb0(%x: f16, %y: f16, %o: f16):
      %v = arith.addf %x, %y : f16
      linalg.yield %v : f16
  } -> tensor<?x?xf16>
  %e1 = tensor.empty(%m, %n) : tensor<?x?xf16>
  %p = linalg.generic {indexing_maps = [#row, #all, #all], iterator_types = ["parallel", "parallel"]}
      ins(%c, %d : tensor<?xf16>, tensor<?x?xf16>) outs(%e1 : tensor<?x?xf16>) {
    ^bb0(%x: f16, %y: f16, %o: f16):
      %v = arith.mulf %x, %y : f16
      linalg.yield %v : f16
  } -> tensor<?x?xf16>
  %out = tensor.concat dim(0) %s, %p : (tensor<?x?xf16>, tensor<?x?xf16>) -> tensor<?x?xf16>
  return %out : tensor<?x?xf16>
}
"""

SPLIT_HALVES = """
#row = affine_map<(d0, d1) -> (d0)>
#col = affine_map<(d0, d1) -> (d1)>
#all = affine_map<(d0, d1) -> (d0, d1)>
func.func @split_halves(%a : tensor<?x?xf16>, %b0 : tensor<?xf16>, %b1 : tensor<?xf16>,
                        %s0 : tensor<?xf16>, %s1 : tensor<?xf16>) -> tensor<?x?xf16> {
  %c0 = arith.constant 0 : index
  %c1 = arith.constant 1 : index
  %z = arith.constant 0.0 : f16
  %n = tensor.dim %a, %c1 : tensor<?x?xf16>
  %h = tensor.dim %b0, %c0 : tensor<?xf16>
  %top = tensor.extract_slice %a[0, 0][%h, %n][1, 1] : tensor<?x?xf16> to tensor<?x?xf16>
  %bot = tensor.extract_slice %a[%h, 0][%h, %n][1, 1] : tensor<?x?xf16> to tensor<?x?xf16>
  %e0 = tensor.empty(%h, %n) : tensor<?x?xf16>
  %o0 = linalg.generic {indexing_maps = [#all, #row, #col, #all], iterator_types = ["parallel", "parallel"]}
      ins(%top, %b0, %s0 : tensor<?x?xf16>, tensor<?xf16>, tensor<?xf16>) outs(%e0 : tensor<?x?xf16>) {
    ^bb0(%x: f16, %b: f16, %s: f16, %o: f16):
      %r = arith.maximumf %x, %z : f16
      %t = arith.addf %r, %b : f16
      %v = arith.mulf %t, %s : f16
      linalg.yield %v : f16
  } -> tensor<?x?xf16>
  %e1 = tensor.empty(%h, %n) : tensor<?x?xf16>
  %o1 = linalg.generic {indexing_maps = [#all, #row, #col, #all], iterator_types = ["parallel", "parallel"]}
      ins(%bot, %b1, %s1 : tensor<?x?xf16>, tensor<?xf16>, tensor<?xf16>) outs(%e1 : tensor<?x?xf16>) {
    ^bb0(%x: f16, %b: f16, %s: f16, %o: f16):
      %r = arith.maximumf %x, %z : f16
      %t = arith.addf %r, %b : f16
      %v = arith.mulf %t, %s : f16
      linalg.yield %v : f16
  } -> tensor<?x?xf16>
  %out = tensor.concat dim(0) %o0, %o1 : (tensor<?x?xf16>, tensor<?x?xf16>) -> tensor<?x?xf16>
  return %out : tensor<?x?xf16>
}
"""

# the five benchmark configurations as linalg graphs ---------------------------

C1_AFIR = """
func.func @add_mul(%arg0: tensor<?x?xf32>, %arg1: tensor<?x?xf32>) -> tensor<?x?xf32> {
  %0 = afir.add %arg0, %arg1 : (tensor<?x?xf32>, tensor<?x?xf32>) -> tensor<?x?xf32>
  %1 = afir.mul %0, %arg1 : (tensor<?x?xf32>, tensor<?x?xf32>) -> tensor<?x?xf32>
  return %1 : tensor<?x?xf32>
}
"""

C2_LINALG = """
#col = affine_map<(d0, d1) -> (d1)>
#row = affine_map<(d0, d1) -> (d0)>
#all = affine_map<(d0, d1) -> (d0, d1)>
func.func @bcast_add_rowsum(%x : tensor<?x?xf32>, %bias : tensor<?xf32>) -> tensor<?xf32> {
  %c0 = arith.constant 0 : index
  %c1 = arith.constant 1 : index
  %m = tensor.dim %x, %c0 : tensor<?x?xf32>
  %n = tensor.dim %x, %c1 : tensor<?x?xf32>
  %e0 = tensor.empty(%m, %n) : tensor<?x?xf32>
  %s = linalg.generic {indexing_maps = [#all, #col, #all], iterator_types = ["parallel", "parallel"]}
      ins(%x, %bias : tensor<?x?xf32>, tensor<?xf32>) outs(%e0 : tensor<?x?xf32>) {
    ^bb0(%a: f32, %b: f32, %o: f32):
      %v = arith.addf %a, %b : f32
      linalg.yield %v : f32
  } -> tensor<?x?xf32>
  %zero = arith.constant 0.0 : f32
  %e1 = tensor.empty(%m) : tensor<?xf32>
  %init = linalg.fill ins(%zero : f32) outs(%e1 : tensor<?xf32>) -> tensor<?xf32>
  %y = linalg.generic {indexing_maps = [#all, #row], iterator_types = ["parallel", "reduction"]}
      ins(%s : tensor<?x?xf32>) outs(%init : tensor<?xf32>) {
    ^bb0(%a: f32, %acc: f32):
      %v = arith.addf %a, %acc : f32
      linalg.yield %v : f32
  } -> tensor<?xf32>
  return %y : tensor<?xf32>
}
"""

C3_LINALG = """
// out[b, j, i] = relu(x[b, i, j]) + c[j]: one parallel generic over the output space
func.func @relu_bcast_transpose(%x : tensor<?x?x?xf16>, %c : tensor<?xf16>) -> tensor<?x?x?xf16> {
  %c0 = arith.constant 0 : index
  %c1 = arith.constant 1 : index
  %c2 = arith.constant 2 : index
  %z = arith.constant 0.0 : f16
  %b = tensor.dim %x, %c0 : tensor<?x?x?xf16>
  %m = tensor.dim %x, %c1 : tensor<?x?x?xf16>
  %n = tensor.dim %x, %c2 : tensor<?x?x?xf16>
  %e = tensor.empty(%b, %n, %m) : tensor<?x?x?xf16>
  %r = linalg.generic {
      indexing_maps = [affine_map<(d0, d1, d2) -> (d0, d2, d1)>, affine_map<(d0, d1, d2) -> (d1)>,
                       affine_map<(d0, d1, d2) -> (d0, d1, d2)>],
      iterator_types = ["parallel", "parallel", "parallel"]
    } ins(%x, %c : tensor<?x?x?xf16>, tensor<?xf16>) outs(%e : tensor<?x?x?xf16>) {
    ^bb0(%v: f16, %k: f16, %o: f16):
      %p = arith.maximumf %v, %z : f16
      %s = arith.addf %p, %k : f16
      linalg.yield %s : f16
  } -> tensor<?x?x?xf16>
  return %r : tensor<?x?x?xf16>
}
"""

C4_LINALG = """
// out[r, :] = table[idx[r], :] * scale + shift
#rowi = affine_map<(d0, d1) -> (d0)>
#col = affine_map<(d0, d1) -> (d1)>
#all = affine_map<(d0, d1) -> (d0, d1)>
func.func @gather_scale_shift(%table : tensor<?x?xf16>, %idx : tensor<?xi32>, %scale : tensor<?xf16>,
                              %shift : tensor<?xf16>) -> tensor<?x?xf16> {
  %c0 = arith.constant 0 : index
  %c1 = arith.constant 1 : index
  %d = tensor.dim %table, %c1 : tensor<?x?xf16>
  %r = tensor.dim %idx, %c0 : tensor<?xi32>
  %e0 = tensor.empty(%r, %d) : tensor<?x?xf16>
  %g = linalg.generic {indexing_maps = [#rowi, #all], iterator_types = ["parallel", "parallel"]}
      ins(%idx : tensor<?xi32>) outs(%e0 : tensor<?x?xf16>) {
    ^bb0(%ix: i32, %o: f16):
      %p = arith.index_cast %ix : i32 to index
      %j = linalg.index 1 : index
      %v = tensor.extract %table[%p, %j] : tensor<?x?xf16>
      linalg.yield %v : f16
  } -> tensor<?x?xf16>
  %e1 = tensor.empty(%r, %d) : tensor<?x?xf16>
  %o = linalg.generic {indexing_maps = [#all, #col, #col, #all], iterator_types = ["parallel", "parallel"]}
      ins(%g, %scale, %shift : tensor<?x?xf16>, tensor<?xf16>, tensor<?xf16>) outs(%e1 : tensor<?x?xf16>) {
    ^bb0(%v: f16, %s: f16, %h: f16, %q: f16):
      %t = arith.mulf %v, %s : f16
      %u = arith.addf %t, %h : f16
      linalg.yield %u : f16
  } -> tensor<?x?xf16>
  return %o : tensor<?x?xf16>
}
"""

# AFIR: implicit numpy broadcast, attributes in the custom syntax, reduction
AFIR_BROADCAST_CHAIN = """
#map3d = affine_map<(d0, d1, d2) -> (d0, d1, d2)>
func.func @bcast_chain(%arg0: tensor<4x1x31xf32>, %arg1: tensor<1x30x1xf32>) -> tensor<?x?x?xf32> {
    %2 = afir.add %arg0, %arg1 : (tensor<4x1x31xf32>, tensor<1x30x1xf32>) -> tensor<?x?x?xf32>
    %3 = afir.mul %2, %arg1 : (tensor<?x?x?xf32>, tensor<1x30x1xf32>) -> tensor<?x?x?xf32>
    %4 = afir.sub %arg1, %3 : (tensor<1x30x1xf32>, tensor<?x?x?xf32>) -> tensor<?x?x?xf32>
    %5 = afir.leaky_relu %4 {indexing_maps = [#map3d, #map3d], negative_slop = 0.01 : f32, outputs = [#afir.asc_tensor<vectorized_axis = [0, 1], vectorized_strides = [4, 1], tensor_id = 0, reuse_id = -1, position = <vector_in, depth = 0, is_double_buffer = false>, position_id = 0>]} : tensor<?x?x?xf32> -> tensor<?x?x?xf32>
    return %5 : tensor<?x?x?xf32>
}
"""

AFIR_DIV_RELU_SUM = """
#map2d = affine_map<(d0, d1) -> (d0, d1)>
#map1d = affine_map<(d0) -> (d0)>
func.func @div_relu_sum(%arg0: tensor<6x40xf32>, %arg1: tensor<40xf32>) -> tensor<6xf32> {
  %0 = afir.broadcast %arg1 {indexing_maps = [#map1d, #map2d]} : tensor<40xf32> -> tensor<6x40xf32>
  %1 = afir.div %arg0, %0 : (tensor<6x40xf32>, tensor<6x40xf32>) -> tensor<6x40xf32>
  %2 = afir.relu %1 {indexing_maps = [#map2d, #map2d]} : tensor<6x40xf32> -> tensor<6x40xf32>
  %3 = afir.sum %2 {indexing_maps = [#map2d, #map1d], axis = 1 : i32} : tensor<6x40xf32> -> tensor<6xf32>
  return %3 : tensor<6xf32>
}
"""


# relu(a - b) * a + (-b) on i32 tensors: the integer side of the AFIR binary / unary math
# ops (include/Dialect/AFIR/Ops/Basic/math.td:71-98), with dynamic shapes.
INT_CHAIN_I32 = """
func.func @int_chain(%a : tensor<?x?xi32>, %b : tensor<?x?xi32>) -> tensor<?x?xi32> {
  %0 = afir.sub %a, %b : (tensor<?x?xi32>, tensor<?x?xi32>) -> tensor<?x?xi32>
  %1 = afir.relu %0 : tensor<?x?xi32> -> tensor<?x?xi32>
  %2 = afir.mul %1, %a : (tensor<?x?xi32>, tensor<?x?xi32>) -> tensor<?x?xi32>
  %3 = afir.neg %b : tensor<?x?xi32> -> tensor<?x?xi32>
  %4 = afir.add %2, %3 : (tensor<?x?xi32>, tensor<?x?xi32>) -> tensor<?x?xi32>
  return %4 : tensor<?x?xi32>
}
"""

# The other matmul-like ops the reference's recogniser takes
# (lib/Conversion/MarkStructuredOps/AnnotateMixMatmulSemanticsPass.cpp:244-256):
# transposed operands and batches.
MATMUL_TRANSPOSE_A_F16 = MATMUL_PLAIN_F16.replace("linalg.matmul ", "linalg.matmul_transpose_a ") \
    .replace("@mm_plain", "@mm_ta")
MATMUL_TRANSPOSE_B_F16 = MATMUL_PLAIN_F16.replace("linalg.matmul ", "linalg.matmul_transpose_b ") \
    .replace("@mm_plain", "@mm_tb")
MATMUL_TRANSPOSE_B_BIAS_LEAKY_BF16 = MATMUL_BIAS_LEAKY_BF16.replace("linalg.matmul ", "linalg.matmul_transpose_b ") \
    .replace("@mm_bias_leaky_bf16", "@mm_tb_bias_leaky_bf16")
BATCH_MATMUL_BF16 = """
func.func @bmm(%a : tensor<?x?x?xbf16>, %b : tensor<?x?x?xbf16>, %init : tensor<?x?x?xbf16>) -> tensor<?x?x?xbf16> {
  %c = linalg.batch_matmul ins(%a, %b : tensor<?x?x?xbf16>, tensor<?x?x?xbf16>)
                           outs(%init : tensor<?x?x?xbf16>) -> tensor<?x?x?xbf16>
  return %c : tensor<?x?x?xbf16>
}
"""
BATCH_MATMUL_TRANSPOSE_B_F16 = BATCH_MATMUL_BF16.replace("xbf16", "xf16").replace("linalg.batch_matmul ", "linalg.batch_matmul_transpose_b ") \
    .replace("outs(%init : tensor<?x?x?xf16>) -> tensor<?x?x?xf16>", "outs(%init : tensor<?x?x?xf32>) -> tensor<?x?x?xf32>") \
    .replace("%init : tensor<?x?x?xf16>) -> tensor<?x?x?xf16> {", "%init : tensor<?x?x?xf32>) -> tensor<?x?x?xf32> {") \
    .replace("return %c : tensor<?x?x?xf16>", "return %c : tensor<?x?x?xf32>").replace("@bmm", "@bmm_tb")

# a mixed-precision chain: f32 values rounded to f16 where the IR says so (arith.truncf), widened
# again (arith.extf, exact) and used in float32 arithmetic:
# out = f16(f32(f16(a)) + f32(b)) * a), a f32 [m, n], b f16 [n]
MIXED_PRECISION_CHAIN = """
func.func @mixed(%a : tensor<?x?xf32>, %b : tensor<?xf16>) -> tensor<?x?xf16> {
  %c0 = arith.constant 0 : index
  %c1 = arith.constant 1 : index
  %m = tensor.dim %a, %c0 : tensor<?x?xf32>
  %n = tensor.dim %a, %c1 : tensor<?x?xf32>
  %e = tensor.empty(%m, %n) : tensor<?x?xf16>
  %o = linalg.generic {indexing_maps = [affine_map<(d0, d1) -> (d0, d1)>, affine_map<(d0, d1) -> (d1)>,
                                        affine_map<(d0, d1) -> (d0, d1)>], iterator_types = ["parallel", "parallel"]}
      ins(%a, %b : tensor<?x?xf32>, tensor<?xf16>) outs(%e : tensor<?x?xf16>) {
    ^bb0(%x: f32, %y: f16, %q: f16):
      %t = arith.truncf %x : f32 to f16
      %tw = arith.extf %t : f16 to f32
      %yw = arith.extf %y : f16 to f32
      %s = arith.addf %tw, %yw : f32
      %v = arith.mulf %s, %x : f32
      %r = arith.truncf %v : f32 to f16
      linalg.yield %r : f16
  } -> tensor<?x?xf16>
  return %o : tensor<?x?xf16>
}
"""

# the named linalg ops and reshapes the reference's --linalg-mark / --linalg-add-broadcast passes
# consume and produce (test/Dialect/AFIR/Transforms/linalgMark.mlir:35-44,
# linalgAddBroadcast.mlir:17-21), and afir.cast between float types
# (include/Dialect/AFIR/Ops/Basic/cast.td:22-25):
# out = bf16((a + transpose(b)) * broadcast(c)) widened to f32, a [4, 8], b [8, 4], c [8]
NAMED_OPS_GRAPH = """
func.func @named(%a : tensor<4x8xf32>, %b : tensor<8x4xf32>, %c : tensor<8xf32>) -> tensor<4x8xf32> {
  %z = arith.constant dense<0.0> : tensor<4x8xf32>
  %e1 = tensor.empty() : tensor<4x8xf32>
  %bt = linalg.transpose ins(%b : tensor<8x4xf32>) outs(%e1 : tensor<4x8xf32>) permutation = [1, 0]
  %s = linalg.add ins(%a, %bt : tensor<4x8xf32>, tensor<4x8xf32>) outs(%z : tensor<4x8xf32>) -> tensor<4x8xf32>
  %e2 = tensor.empty() : tensor<4x8xf32>
  %cb = linalg.broadcast ins(%c : tensor<8xf32>) outs(%e2 : tensor<4x8xf32>) dimensions = [0]
  %m = linalg.mul ins(%s, %cb : tensor<4x8xf32>, tensor<4x8xf32>) outs(%z : tensor<4x8xf32>) -> tensor<4x8xf32>
  %x = tensor.expand_shape %m [[0, 1], [2]] output_shape [4, 1, 8] : tensor<4x8xf32> into tensor<4x1x8xf32>
  %y = tensor.collapse_shape %x [[0, 1], [2]] : tensor<4x1x8xf32> into tensor<4x8xf32>
  %r = afir.cast %y : tensor<4x8xf32> -> tensor<4x8xbf16>
  %w = afir.cast %r : tensor<4x8xbf16> -> tensor<4x8xf32>
  return %w : tensor<4x8xf32>
}
"""

# linalg.elementwise with broadcast maps, dynamic shapes: out[i, j, k] = a[j, k] - c[i, 0, k]
ELEMENTWISE_KIND_SUB = """
func.func @ew_sub(%a : tensor<?x?xf16>, %c : tensor<?x1x?xf16>, %init : tensor<?x?x?xf16>) -> tensor<?x?x?xf16> {
  %r = linalg.elementwise kind=#linalg.elementwise_kind<sub>
      indexing_maps = [affine_map<(d0, d1, d2) -> (d1, d2)>, affine_map<(d0, d1, d2) -> (d0, 0, d2)>,
                       affine_map<(d0, d1, d2) -> (d0, d1, d2)>]
      ins(%a, %c : tensor<?x?xf16>, tensor<?x1x?xf16>) outs(%init : tensor<?x?x?xf16>) -> tensor<?x?x?xf16>
  return %r : tensor<?x?x?xf16>
}
"""


# A row sum written with named ops only: linalg.square / broadcast / add / reciprocal / copy and
# linalg.reduce with an addf combiner over the innermost dim (the op names of the reference's
# --linalg-mark groups 1 and 2, lib/Dialect/AFIR/Transforms/LinalgMark.cpp:45-62):
# y[i] = sum_j 1 / (x[i,j]^2 + b[j])
NAMED_REDUCE_GRAPH = """
func.func @sq_recip_rowsum(%x: tensor<?x?xf32>, %b: tensor<?xf32>) -> tensor<?xf32> {
  %c0 = arith.constant 0 : index
  %c1 = arith.constant 1 : index
  %m = tensor.dim %x, %c0 : tensor<?x?xf32>
  %n = tensor.dim %x, %c1 : tensor<?x?xf32>
  %e = tensor.empty(%m, %n) : tensor<?x?xf32>
  %sq = linalg.square ins(%x : tensor<?x?xf32>) outs(%e : tensor<?x?xf32>) -> tensor<?x?xf32>
  %bb = linalg.broadcast ins(%b : tensor<?xf32>) outs(%e : tensor<?x?xf32>) dimensions = [0]
  %s = linalg.add ins(%sq, %bb : tensor<?x?xf32>, tensor<?x?xf32>) outs(%e : tensor<?x?xf32>) -> tensor<?x?xf32>
  %r = linalg.reciprocal ins(%s : tensor<?x?xf32>) outs(%e : tensor<?x?xf32>) -> tensor<?x?xf32>
  %cp = linalg.copy ins(%r : tensor<?x?xf32>) outs(%e : tensor<?x?xf32>) -> tensor<?x?xf32>
  %zero = arith.constant 0.0 : f32
  %ie = tensor.empty(%m) : tensor<?xf32>
  %init = linalg.fill ins(%zero : f32) outs(%ie : tensor<?xf32>) -> tensor<?xf32>
  %red = linalg.reduce ins(%cp : tensor<?x?xf32>) outs(%init : tensor<?xf32>) dimensions = [1]
    (%in: f32, %acc: f32) {
      %0 = arith.addf %in, %acc : f32
      linalg.yield %0 : f32
    }
  return %red : tensor<?xf32>
}
"""
