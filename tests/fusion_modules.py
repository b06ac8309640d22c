"""Decomposed StableHLO modules (the forms JAX-style lowering produces, which the
reference's pattern detectors accept: Optimizer/FusionPatterns.swift:18-1142) shared by
the CPU and GPU fusion tests."""

SOFTMAX = """func.func @main(%x: tensor<8x32xf32>) -> tensor<8x32xf32> {
  %ninf = stablehlo.constant dense<0xFF800000> : tensor<f32>
  %m = stablehlo.reduce(%x init: %ninf) applies stablehlo.maximum across dimensions = [1] : (tensor<8x32xf32>, tensor<f32>) -> tensor<8xf32>
  %mb = stablehlo.broadcast_in_dim %m, dims = [0] : (tensor<8xf32>) -> tensor<8x32xf32>
  %sh = stablehlo.subtract %x, %mb : tensor<8x32xf32>
  %e = stablehlo.exponential %sh : tensor<8x32xf32>
  %zero = stablehlo.constant dense<0.0> : tensor<f32>
  %s = stablehlo.reduce(%e init: %zero) applies stablehlo.add across dimensions = [1] : (tensor<8x32xf32>, tensor<f32>) -> tensor<8xf32>
  %sb = stablehlo.broadcast_in_dim %s, dims = [0] : (tensor<8xf32>) -> tensor<8x32xf32>
  %r = stablehlo.divide %e, %sb : tensor<8x32xf32>
  return %r : tensor<8x32xf32> }"""

# the same chain, but the exponentials are also returned: an interior value escapes
SOFTMAX_ESCAPING = SOFTMAX.replace("-> tensor<8x32xf32> {", "-> (tensor<8x32xf32>, tensor<8x32xf32>) {") \
                          .replace("return %r : tensor<8x32xf32>", "return %r, %e : tensor<8x32xf32>, tensor<8x32xf32>")

SOFTMAX_AXIS0 = """func.func @main(%x: tensor<8x32xf32>) -> tensor<8x32xf32> {
  %ninf = stablehlo.constant dense<0xFF800000> : tensor<f32>
  %m = stablehlo.reduce(%x init: %ninf) applies stablehlo.maximum across dimensions = [0] : (tensor<8x32xf32>, tensor<f32>) -> tensor<32xf32>
  %mb = stablehlo.broadcast_in_dim %m, dims = [1] : (tensor<32xf32>) -> tensor<8x32xf32>
  %sh = stablehlo.subtract %x, %mb : tensor<8x32xf32>
  %e = stablehlo.exponential %sh : tensor<8x32xf32>
  %zero = stablehlo.constant dense<0.0> : tensor<f32>
  %s = stablehlo.reduce(%e init: %zero) applies stablehlo.add across dimensions = [0] : (tensor<8x32xf32>, tensor<f32>) -> tensor<32xf32>
  %sb = stablehlo.broadcast_in_dim %s, dims = [1] : (tensor<32xf32>) -> tensor<8x32xf32>
  %r = stablehlo.divide %e, %sb : tensor<8x32xf32>
  return %r : tensor<8x32xf32> }"""

GELU = """func.func @main(%x: tensor<4x64xf32>) -> tensor<4x64xf32> {
  %half = stablehlo.constant dense<0.5> : tensor<4x64xf32>
  %one = stablehlo.constant dense<1.0> : tensor<4x64xf32>
  %coeff = stablehlo.constant dense<0.044715> : tensor<4x64xf32>
  %k = stablehlo.constant dense<0.7978845608> : tensor<4x64xf32>
  %x2 = stablehlo.multiply %x, %x : tensor<4x64xf32>
  %x3 = stablehlo.multiply %x2, %x : tensor<4x64xf32>
  %cx3 = stablehlo.multiply %coeff, %x3 : tensor<4x64xf32>
  %inner = stablehlo.add %x, %cx3 : tensor<4x64xf32>
  %sc = stablehlo.multiply %k, %inner : tensor<4x64xf32>
  %t = stablehlo.tanh %sc : tensor<4x64xf32>
  %opt = stablehlo.add %one, %t : tensor<4x64xf32>
  %hx = stablehlo.multiply %half, %x : tensor<4x64xf32>
  %r = stablehlo.multiply %hx, %opt : tensor<4x64xf32>
  return %r : tensor<4x64xf32> }"""

# wrong cubic coefficient: not GELU, must stay as written
NOT_GELU = GELU.replace("0.044715", "0.144715")

LAYER_NORM = """func.func @main(%x: tensor<16x64xf32>, %g: tensor<64xf32>, %b: tensor<64xf32>) -> tensor<16x64xf32> {
  %zero = stablehlo.constant dense<0.0> : tensor<f32>
  %n = stablehlo.constant dense<64.0> : tensor<16xf32>
  %eps = stablehlo.constant dense<1.0e-5> : tensor<16xf32>
  %s = stablehlo.reduce(%x init: %zero) applies stablehlo.add across dimensions = [1] : (tensor<16x64xf32>, tensor<f32>) -> tensor<16xf32>
  %mean = stablehlo.divide %s, %n : tensor<16xf32>
  %mb = stablehlo.broadcast_in_dim %mean, dims = [0] : (tensor<16xf32>) -> tensor<16x64xf32>
  %c = stablehlo.subtract %x, %mb : tensor<16x64xf32>
  %sq = stablehlo.multiply %c, %c : tensor<16x64xf32>
  %s2 = stablehlo.reduce(%sq init: %zero) applies stablehlo.add across dimensions = [1] : (tensor<16x64xf32>, tensor<f32>) -> tensor<16xf32>
  %var = stablehlo.divide %s2, %n : tensor<16xf32>
  %ve = stablehlo.add %var, %eps : tensor<16xf32>
  %r = stablehlo.rsqrt %ve : tensor<16xf32>
  %rb = stablehlo.broadcast_in_dim %r, dims = [0] : (tensor<16xf32>) -> tensor<16x64xf32>
  %xn = stablehlo.multiply %c, %rb : tensor<16x64xf32>
  %gb = stablehlo.broadcast_in_dim %g, dims = [1] : (tensor<64xf32>) -> tensor<16x64xf32>
  %bb = stablehlo.broadcast_in_dim %b, dims = [1] : (tensor<64xf32>) -> tensor<16x64xf32>
  %y = stablehlo.multiply %xn, %gb : tensor<16x64xf32>
  %z = stablehlo.add %y, %bb : tensor<16x64xf32>
  return %z : tensor<16x64xf32> }"""

RMS_NORM = """func.func @main(%x: tensor<16x64xf32>, %g: tensor<64xf32>) -> tensor<16x64xf32> {
  %zero = stablehlo.constant dense<0.0> : tensor<f32>
  %rn = stablehlo.constant dense<0.015625> : tensor<16xf32>
  %eps = stablehlo.constant dense<1.0e-6> : tensor<16xf32>
  %sq = stablehlo.multiply %x, %x : tensor<16x64xf32>
  %s2 = stablehlo.reduce(%sq init: %zero) applies stablehlo.add across dimensions = [1] : (tensor<16x64xf32>, tensor<f32>) -> tensor<16xf32>
  %ms = stablehlo.multiply %s2, %rn : tensor<16xf32>
  %ve = stablehlo.add %ms, %eps : tensor<16xf32>
  %r = stablehlo.rsqrt %ve : tensor<16xf32>
  %rb = stablehlo.broadcast_in_dim %r, dims = [0] : (tensor<16xf32>) -> tensor<16x64xf32>
  %xn = stablehlo.multiply %x, %rb : tensor<16x64xf32>
  %gb = stablehlo.broadcast_in_dim %g, dims = [1] : (tensor<64xf32>) -> tensor<16x64xf32>
  %y = stablehlo.multiply %gb, %xn : tensor<16x64xf32>
  return %y : tensor<16x64xf32> }"""


def attention(B=2, H=3, S=64, D=32, with_mask=False, transpose_k=True, divide=False, dtype="f32"):
    t = f"tensor<{B}x{H}x{S}x{D}x{dtype}>"
    st = f"tensor<{B}x{H}x{S}x{S}x{dtype}>"
    rt = f"tensor<{B}x{H}x{S}x{dtype}>"
    args = f"%q: {t}, %k: {t}, %v: {t}" + (f", %mask: tensor<{S}x{S}x{dtype}>" if with_mask else "")
    lines = [f"func.func @main({args}) -> {t} {{"]
    if transpose_k:
        kt = f"tensor<{B}x{H}x{D}x{S}x{dtype}>"
        lines.append(f"  %kt = stablehlo.transpose %k, dims = [0, 1, 3, 2] : ({t}) -> {kt}")
        lines.append(f"  %s0 = stablehlo.dot_general %q, %kt, batching_dims = [0, 1] x [0, 1], contracting_dims = [3] x [2] : ({t}, {kt}) -> {st}")
    else:
        lines.append(f"  %s0 = stablehlo.dot_general %q, %k, batching_dims = [0, 1] x [0, 1], contracting_dims = [3] x [3] : ({t}, {t}) -> {st}")
    if divide:
        lines.append(f"  %sc = stablehlo.constant dense<{D ** 0.5!r}> : {st}")
        lines.append(f"  %s1 = stablehlo.divide %s0, %sc : {st}")
    else:
        lines.append(f"  %sc = stablehlo.constant dense<{D ** -0.5!r}> : {st}")
        lines.append(f"  %s1 = stablehlo.multiply %s0, %sc : {st}")
    cur = "%s1"
    if with_mask:
        lines.append(f"  %mbc = stablehlo.broadcast_in_dim %mask, dims = [2, 3] : (tensor<{S}x{S}x{dtype}>) -> {st}")
        lines.append(f"  %s2 = stablehlo.add %s1, %mbc : {st}")
        cur = "%s2"
    neg = {"f32": "0xFF800000", "bf16": "0xFF80", "f16": "0xFC00"}[dtype]
    lines += [
        f"  %ninf = stablehlo.constant dense<{neg}> : tensor<{dtype}>",
        f"  %zero = stablehlo.constant dense<0.0> : tensor<{dtype}>",
        f"  %m = stablehlo.reduce({cur} init: %ninf) applies stablehlo.maximum across dimensions = [3] : ({st}, tensor<{dtype}>) -> {rt}",
        f"  %mb = stablehlo.broadcast_in_dim %m, dims = [0, 1, 2] : ({rt}) -> {st}",
        f"  %sh = stablehlo.subtract {cur}, %mb : {st}",
        f"  %e = stablehlo.exponential %sh : {st}",
        f"  %s = stablehlo.reduce(%e init: %zero) applies stablehlo.add across dimensions = [3] : ({st}, tensor<{dtype}>) -> {rt}",
        f"  %sb = stablehlo.broadcast_in_dim %s, dims = [0, 1, 2] : ({rt}) -> {st}",
        f"  %p = stablehlo.divide %e, %sb : {st}",
        f"  %o = stablehlo.dot_general %p, %v, batching_dims = [0, 1] x [0, 1], contracting_dims = [3] x [2] : ({st}, {t}) -> {t}",
        f"  return %o : {t} }}"]
    return "\n".join(lines)


FFN_UP = """func.func @main(%x: tensor<32x64xf32>, %w: tensor<64x128xf32>, %b: tensor<128xf32>) -> tensor<32x128xf32> {
  %d = stablehlo.dot_general %x, %w, contracting_dims = [1] x [0] : (tensor<32x64xf32>, tensor<64x128xf32>) -> tensor<32x128xf32>
  %bb = stablehlo.broadcast_in_dim %b, dims = [1] : (tensor<128xf32>) -> tensor<32x128xf32>
  %h = stablehlo.add %d, %bb : tensor<32x128xf32>
  %half = stablehlo.constant dense<0.5> : tensor<32x128xf32>
  %one = stablehlo.constant dense<1.0> : tensor<32x128xf32>
  %coeff = stablehlo.constant dense<0.044715> : tensor<32x128xf32>
  %k = stablehlo.constant dense<0.7978845608> : tensor<32x128xf32>
  %h2 = stablehlo.multiply %h, %h : tensor<32x128xf32>
  %h3 = stablehlo.multiply %h, %h2 : tensor<32x128xf32>
  %ch3 = stablehlo.multiply %h3, %coeff : tensor<32x128xf32>
  %inner = stablehlo.add %ch3, %h : tensor<32x128xf32>
  %sc = stablehlo.multiply %inner, %k : tensor<32x128xf32>
  %t = stablehlo.tanh %sc : tensor<32x128xf32>
  %opt = stablehlo.add %t, %one : tensor<32x128xf32>
  %xo = stablehlo.multiply %h, %opt : tensor<32x128xf32>
  %r = stablehlo.multiply %half, %xo : tensor<32x128xf32>
  return %r : tensor<32x128xf32> }"""

MATMUL_BIAS_RELU = """func.func @main(%x: tensor<32x64xf32>, %w: tensor<64x128xf32>, %b: tensor<128xf32>) -> tensor<32x128xf32> {
  %d = stablehlo.dot %x, %w : (tensor<32x64xf32>, tensor<64x128xf32>) -> tensor<32x128xf32>
  %bb = stablehlo.broadcast_in_dim %b, dims = [1] : (tensor<128xf32>) -> tensor<32x128xf32>
  %h = stablehlo.add %bb, %d : tensor<32x128xf32>
  %zero = stablehlo.constant dense<0.0> : tensor<32x128xf32>
  %r = stablehlo.maximum %h, %zero : tensor<32x128xf32>
  return %r : tensor<32x128xf32> }"""

# keepdims style, as array libraries write `x - max(x, axis, keepdims=True)`: the statistic is
# renamed to a shape with a unit dim (broadcast_in_dim or reshape), possibly computed on there,
# and spread over the row by a second broadcast
SOFTMAX_KEEPDIMS = """module @jit_softmax attributes {mhlo.num_partitions = 1 : i32, mhlo.num_replicas = 1 : i32} {
  func.func public @main(%arg0: tensor<8x32xf32> {mhlo.layout_mode = "default"}) -> (tensor<8x32xf32> {jax.result_info = "", mhlo.layout_mode = "default"}) {
    %cst = stablehlo.constant dense<0xFF800000> : tensor<f32>
    %0 = stablehlo.reduce(%arg0 init: %cst) applies stablehlo.maximum across dimensions = [1] : (tensor<8x32xf32>, tensor<f32>) -> tensor<8xf32>
    %1 = stablehlo.broadcast_in_dim %0, dims = [0] : (tensor<8xf32>) -> tensor<8x1xf32>
    %2 = stablehlo.broadcast_in_dim %1, dims = [0, 1] : (tensor<8x1xf32>) -> tensor<8x32xf32>
    %3 = stablehlo.subtract %arg0, %2 : tensor<8x32xf32>
    %4 = stablehlo.exponential %3 : tensor<8x32xf32>
    %cst_0 = stablehlo.constant dense<0.000000e+00> : tensor<f32>
    %5 = stablehlo.reduce(%4 init: %cst_0) applies stablehlo.add across dimensions = [1] : (tensor<8x32xf32>, tensor<f32>) -> tensor<8xf32>
    %6 = stablehlo.reshape %5 : (tensor<8xf32>) -> tensor<8x1xf32>
    %7 = stablehlo.broadcast_in_dim %6, dims = [0, 1] : (tensor<8x1xf32>) -> tensor<8x32xf32>
    %8 = stablehlo.divide %4, %7 : tensor<8x32xf32>
    return %8 : tensor<8x32xf32>
  }
}"""

LAYER_NORM_KEEPDIMS = """func.func @main(%x: tensor<16x64xf32>, %g: tensor<64xf32>, %b: tensor<64xf32>) -> tensor<16x64xf32> {
  %zero = stablehlo.constant dense<0.0> : tensor<f32>
  %n = stablehlo.constant dense<64.0> : tensor<16xf32>
  %n1 = stablehlo.constant dense<64.0> : tensor<16x1xf32>
  %eps = stablehlo.constant dense<1.0e-5> : tensor<16x1xf32>
  %s = stablehlo.reduce(%x init: %zero) applies stablehlo.add across dimensions = [1] : (tensor<16x64xf32>, tensor<f32>) -> tensor<16xf32>
  %mean = stablehlo.divide %s, %n : tensor<16xf32>
  %mk = stablehlo.broadcast_in_dim %mean, dims = [0] : (tensor<16xf32>) -> tensor<16x1xf32>
  %mb = stablehlo.broadcast_in_dim %mk, dims = [0, 1] : (tensor<16x1xf32>) -> tensor<16x64xf32>
  %c = stablehlo.subtract %x, %mb : tensor<16x64xf32>
  %sq = stablehlo.multiply %c, %c : tensor<16x64xf32>
  %s2 = stablehlo.reduce(%sq init: %zero) applies stablehlo.add across dimensions = [1] : (tensor<16x64xf32>, tensor<f32>) -> tensor<16xf32>
  %s2k = stablehlo.reshape %s2 : (tensor<16xf32>) -> tensor<16x1xf32>
  %var = stablehlo.divide %s2k, %n1 : tensor<16x1xf32>
  %ve = stablehlo.add %var, %eps : tensor<16x1xf32>
  %r = stablehlo.rsqrt %ve : tensor<16x1xf32>
  %rb = stablehlo.broadcast_in_dim %r, dims = [0, 1] : (tensor<16x1xf32>) -> tensor<16x64xf32>
  %xn = stablehlo.multiply %c, %rb : tensor<16x64xf32>
  %gb = stablehlo.broadcast_in_dim %g, dims = [1] : (tensor<64xf32>) -> tensor<16x64xf32>
  %bb = stablehlo.broadcast_in_dim %b, dims = [1] : (tensor<64xf32>) -> tensor<16x64xf32>
  %y = stablehlo.multiply %xn, %gb : tensor<16x64xf32>
  %z = stablehlo.add %y, %bb : tensor<16x64xf32>
  return %z : tensor<16x64xf32> }"""

# the unit dim is put in front and the values are spread over axis 0: a column statistic, not a
# row statistic -- must not be taken for the softmax over axis 1
NOT_SOFTMAX_WRONG_SPREAD = """func.func @main(%x: tensor<8x8xf32>) -> tensor<8x8xf32> {
  %ninf = stablehlo.constant dense<0xFF800000> : tensor<f32>
  %zero = stablehlo.constant dense<0.0> : tensor<f32>
  %m = stablehlo.reduce(%x init: %ninf) applies stablehlo.maximum across dimensions = [1] : (tensor<8x8xf32>, tensor<f32>) -> tensor<8xf32>
  %mk = stablehlo.reshape %m : (tensor<8xf32>) -> tensor<1x8xf32>
  %mb = stablehlo.broadcast_in_dim %mk, dims = [0, 1] : (tensor<1x8xf32>) -> tensor<8x8xf32>
  %sh = stablehlo.subtract %x, %mb : tensor<8x8xf32>
  %e = stablehlo.exponential %sh : tensor<8x8xf32>
  %s = stablehlo.reduce(%e init: %zero) applies stablehlo.add across dimensions = [1] : (tensor<8x8xf32>, tensor<f32>) -> tensor<8xf32>
  %sk = stablehlo.reshape %s : (tensor<8xf32>) -> tensor<1x8xf32>
  %sb = stablehlo.broadcast_in_dim %sk, dims = [0, 1] : (tensor<1x8xf32>) -> tensor<8x8xf32>
  %y = stablehlo.divide %e, %sb : tensor<8x8xf32>
  return %y : tensor<8x8xf32> }"""


from metalhlo_amd.programs import GPT2_LAYER_PARAMS, gpt2_program, transformer_block   # noqa: E402,F401


def masked_attention(form, B=2, H=2, S=64, D=32, dtype="f32"):
    """Attention whose additive [S, S] mask is built in the program from two iotas.  `form`:
    "le" keep where key <= query (compare LE key, query); "ge_swapped" the same written GE query, key;
    "gt_drop" select(key > query, -inf, 0); "big_negative" -1e30 in place of -inf;
    "anti" keep where key >= query (NOT causal); "keep_one" adds 1 where kept (NOT a pure mask)."""
    t, st, rt = f"tensor<{B}x{H}x{S}x{D}x{dtype}>", f"tensor<{B}x{H}x{S}x{S}x{dtype}>", f"tensor<{B}x{H}x{S}x{dtype}>"
    it, mt = f"tensor<{S}x{S}xi32>", f"tensor<{S}x{S}x{dtype}>"
    neg = {"f32": "0xFF800000", "bf16": "0xFF80", "f16": "0xFC00"}[dtype]
    cmp_line, sel = {
        "le": ("LE, %ki, %qi", "%mz, %mn"), "ge_swapped": ("GE, %qi, %ki", "%mz, %mn"), "gt_drop": ("GT, %ki, %qi", "%mn, %mz"),
        "big_negative": ("LE, %ki, %qi", "%mz, %mn"), "anti": ("GE, %ki, %qi", "%mz, %mn"), "keep_one": ("LE, %ki, %qi", "%mz, %mn"),
    }[form]
    drop = "-1.0e30" if form == "big_negative" else neg
    keep = "1.0" if form == "keep_one" else "0.0"
    return "\n".join([
        f"func.func @main(%q: {t}, %k: {t}, %v: {t}) -> {t} {{",
        f"  %s0 = stablehlo.dot_general %q, %k, batching_dims = [0, 1] x [0, 1], contracting_dims = [3] x [3] : ({t}, {t}) -> {st}",
        f"  %sc = stablehlo.constant dense<{D ** -0.5!r}> : {st}",
        f"  %s1 = stablehlo.multiply %s0, %sc : {st}",
        f"  %qi = stablehlo.iota dim = 0 : {it}",
        f"  %ki = stablehlo.iota dim = 1 : {it}",
        f"  %pred = stablehlo.compare {cmp_line}, SIGNED : ({it}, {it}) -> tensor<{S}x{S}xi1>",
        f"  %mz = stablehlo.constant dense<{keep}> : {mt}",
        f"  %mn = stablehlo.constant dense<{drop}> : {mt}",
        f"  %mask = stablehlo.select %pred, {sel} : tensor<{S}x{S}xi1>, {mt}",
        f"  %mbc = stablehlo.broadcast_in_dim %mask, dims = [2, 3] : ({mt}) -> {st}",
        f"  %s2 = stablehlo.add %s1, %mbc : {st}",
        f"  %ninf = stablehlo.constant dense<{neg}> : tensor<{dtype}>",
        f"  %zero = stablehlo.constant dense<0.0> : tensor<{dtype}>",
        f"  %m = stablehlo.reduce(%s2 init: %ninf) applies stablehlo.maximum across dimensions = [3] : ({st}, tensor<{dtype}>) -> {rt}",
        f"  %mb = stablehlo.broadcast_in_dim %m, dims = [0, 1, 2] : ({rt}) -> {st}",
        f"  %sh = stablehlo.subtract %s2, %mb : {st}",
        f"  %e = stablehlo.exponential %sh : {st}",
        f"  %s = stablehlo.reduce(%e init: %zero) applies stablehlo.add across dimensions = [3] : ({st}, tensor<{dtype}>) -> {rt}",
        f"  %sb = stablehlo.broadcast_in_dim %s, dims = [0, 1, 2] : ({rt}) -> {st}",
        f"  %p = stablehlo.divide %e, %sb : {st}",
        f"  %o = stablehlo.dot_general %p, %v, batching_dims = [0, 1] x [0, 1], contracting_dims = [3] x [2] : ({st}, {t}) -> {t}",
        f"  return %o : {t} }}"])


# exact GELU the way jax.nn.gelu(approximate=False) lowers it: x * (erf(x / sqrt 2) + 1) / 2
GELU_ERF = """func.func @main(%x: tensor<4x64xf32>) -> tensor<4x64xf32> {
  %rt2 = stablehlo.constant dense<1.41421354> : tensor<4x64xf32>
  %one = stablehlo.constant dense<1.0> : tensor<4x64xf32>
  %two = stablehlo.constant dense<2.0> : tensor<4x64xf32>
  %u = stablehlo.divide %x, %rt2 : tensor<4x64xf32>
  %e = chlo.erf %u : tensor<4x64xf32> -> tensor<4x64xf32>
  %p = stablehlo.add %e, %one : tensor<4x64xf32>
  %xp = stablehlo.multiply %x, %p : tensor<4x64xf32>
  %r = stablehlo.divide %xp, %two : tensor<4x64xf32>
  return %r : tensor<4x64xf32> }"""

# the other common spelling: 0.5 * x * (1 + erf(x * 0.70710678))
GELU_ERF_MUL = """func.func @main(%x: tensor<4x64xf32>) -> tensor<4x64xf32> {
  %k = stablehlo.constant dense<0.707106769> : tensor<4x64xf32>
  %one = stablehlo.constant dense<1.0> : tensor<4x64xf32>
  %half = stablehlo.constant dense<0.5> : tensor<4x64xf32>
  %u = stablehlo.multiply %x, %k : tensor<4x64xf32>
  %e = chlo.erf %u : tensor<4x64xf32> -> tensor<4x64xf32>
  %p = stablehlo.add %one, %e : tensor<4x64xf32>
  %hx = stablehlo.multiply %half, %x : tensor<4x64xf32>
  %r = stablehlo.multiply %hx, %p : tensor<4x64xf32>
  return %r : tensor<4x64xf32> }"""

# LayerNorm with the one-pass variance mean(x^2) - mean(x)^2 (flax use_fast_variance, jnp.var)
LAYER_NORM_ONE_PASS = """func.func @main(%x: tensor<16x64xf32>, %g: tensor<64xf32>, %b: tensor<64xf32>) -> tensor<16x64xf32> {
  %zero = stablehlo.constant dense<0.0> : tensor<f32>
  %n = stablehlo.constant dense<64.0> : tensor<16xf32>
  %eps = stablehlo.constant dense<1.0e-5> : tensor<16xf32>
  %s = stablehlo.reduce(%x init: %zero) applies stablehlo.add across dimensions = [1] : (tensor<16x64xf32>, tensor<f32>) -> tensor<16xf32>
  %mean = stablehlo.divide %s, %n : tensor<16xf32>
  %xx = stablehlo.multiply %x, %x : tensor<16x64xf32>
  %s2 = stablehlo.reduce(%xx init: %zero) applies stablehlo.add across dimensions = [1] : (tensor<16x64xf32>, tensor<f32>) -> tensor<16xf32>
  %m2 = stablehlo.divide %s2, %n : tensor<16xf32>
  %mm = stablehlo.multiply %mean, %mean : tensor<16xf32>
  %var = stablehlo.subtract %m2, %mm : tensor<16xf32>
  %ve = stablehlo.add %var, %eps : tensor<16xf32>
  %r = stablehlo.rsqrt %ve : tensor<16xf32>
  %mb = stablehlo.broadcast_in_dim %mean, dims = [0] : (tensor<16xf32>) -> tensor<16x64xf32>
  %c = stablehlo.subtract %x, %mb : tensor<16x64xf32>
  %rb = stablehlo.broadcast_in_dim %r, dims = [0] : (tensor<16xf32>) -> tensor<16x64xf32>
  %xn = stablehlo.multiply %c, %rb : tensor<16x64xf32>
  %gb = stablehlo.broadcast_in_dim %g, dims = [1] : (tensor<64xf32>) -> tensor<16x64xf32>
  %bb = stablehlo.broadcast_in_dim %b, dims = [1] : (tensor<64xf32>) -> tensor<16x64xf32>
  %y = stablehlo.multiply %xn, %gb : tensor<16x64xf32>
  %z = stablehlo.add %y, %bb : tensor<16x64xf32>
  return %z : tensor<16x64xf32> }"""

# a module the way a tracing front end writes it: private helpers, a call with two results
# used as %r#0 / %r#1, a call nested inside a callee, the entry function not first
CALLS = """module @jit_f {
  func.func private @_where(%p: tensor<8x16xi1>, %a: tensor<8x16xf32>, %b: tensor<8x16xf32>) -> tensor<8x16xf32> {
    %0 = stablehlo.select %p, %a, %b : tensor<8x16xi1>, tensor<8x16xf32>
    return %0 : tensor<8x16xf32>
  }
  func.func private @relu_and_neg(%a: tensor<8x16xf32>) -> (tensor<8x16xf32>, tensor<8x16xf32>) {
    %z = stablehlo.constant dense<0.0> : tensor<8x16xf32>
    %p = stablehlo.compare GT, %a, %z, FLOAT : (tensor<8x16xf32>, tensor<8x16xf32>) -> tensor<8x16xi1>
    %r = func.call @_where(%p, %a, %z) : (tensor<8x16xi1>, tensor<8x16xf32>, tensor<8x16xf32>) -> tensor<8x16xf32>
    %n = stablehlo.negate %a : tensor<8x16xf32>
    return %r, %n : tensor<8x16xf32>, tensor<8x16xf32>
  }
  func.func public @main(%x: tensor<8x16xf32>, %y: tensor<8x16xf32>) -> (tensor<8x16xf32>, tensor<8x16xf32>) {
    %s = stablehlo.add %x, %y : tensor<8x16xf32>
    %r:2 = call @relu_and_neg(%s) : (tensor<8x16xf32>) -> (tensor<8x16xf32>, tensor<8x16xf32>)
    %t = stablehlo.multiply %r#0, %r#1 : tensor<8x16xf32>
    %u = call @_where_wrapper(%r#1, %t) : (tensor<8x16xf32>, tensor<8x16xf32>) -> tensor<8x16xf32>
    return %t, %u : tensor<8x16xf32>, tensor<8x16xf32>
  }
  func.func private @_where_wrapper(%a: tensor<8x16xf32>, %b: tensor<8x16xf32>) -> tensor<8x16xf32> {
    %z = stablehlo.constant dense<0.0> : tensor<8x16xf32>
    %p = stablehlo.compare LT, %a, %z, FLOAT : (tensor<8x16xf32>, tensor<8x16xf32>) -> tensor<8x16xi1>
    %r = call @_where(%p, %a, %b) : (tensor<8x16xi1>, tensor<8x16xf32>, tensor<8x16xf32>) -> tensor<8x16xf32>
    return %r : tensor<8x16xf32>
  }
}"""

# softmax computed by a helper function: after inlining it is the ordinary pattern
SOFTMAX_IN_CALLEE = """module {
  func.func @main(%x: tensor<8x32xf32>) -> tensor<8x32xf32> {
    %y = call @softmax(%x) : (tensor<8x32xf32>) -> tensor<8x32xf32>
    return %y : tensor<8x32xf32>
  }
""" + SOFTMAX.replace("func.func @main", "  func.func private @softmax") + "\n}"

FFN_CUSTOM_CALL = """func.func @main(%x: tensor<4x32x64xf32>, %up: tensor<64x256xf32>, %down: tensor<256x64xf32>) -> tensor<4x32x64xf32> {
  %r = stablehlo.custom_call @fused_ffn(%x, %up, %down) {backend_config = "{\\"activation\\": \\"ACT\\"}"} : (tensor<4x32x64xf32>, tensor<64x256xf32>, tensor<256x64xf32>) -> tensor<4x32x64xf32>
  return %r : tensor<4x32x64xf32> }"""


def embedding(B=2, S=16, d=64, vocab=50, n_pos=24, dtype="bf16", first=0, ids_type="i32", keep_tokens=False, cols=None):
    """Token gather + positions [first, first+S) of a longer table, repeated over the batch, summed
    in f32 and (for a 16-bit `dtype`) rounded once.  `keep_tokens` also returns the gathered rows;
    `cols` slices fewer columns of a wider position table (not whole rows)."""
    x3f, out_t = f"tensor<{B}x{S}x{d}xf32>", f"tensor<{B}x{S}x{d}x{dtype}>"
    wp = cols or d
    res = f"({out_t}, {x3f})" if keep_tokens else out_t
    L = [f"func.func @main(%ids: tensor<{B}x{S}x{ids_type}>, %wte: tensor<{vocab}x{d}xf32>, %wpe: tensor<{n_pos}x{wp}xf32>) -> {res} {{",
         f'  %tok = "stablehlo.gather"(%wte, %ids) {{ dimension_numbers = #stablehlo.gather<offset_dims = [2], collapsed_slice_dims = [0], '
         f'start_index_map = [0], index_vector_dim = 2>, slice_sizes = array<i64: 1, {d}>, indices_are_sorted = false }} '
         f": (tensor<{vocab}x{d}xf32>, tensor<{B}x{S}x{ids_type}>) -> {x3f}",
         f"  %pos = stablehlo.slice %wpe [{first}:{first + S}, 0:{d}] : (tensor<{n_pos}x{wp}xf32>) -> tensor<{S}x{d}xf32>",
         f"  %posb = stablehlo.broadcast_in_dim %pos, dims = [1, 2] : (tensor<{S}x{d}xf32>) -> {x3f}",
         f"  %emb = stablehlo.add %posb, %tok : {x3f}"]
    last = "%emb"
    if dtype != "f32":
        L.append(f"  %h = stablehlo.convert %emb : ({x3f}) -> {out_t}")
        last = "%h"
    L.append(f"  return {last}, %tok : {out_t}, {x3f} }}" if keep_tokens else f"  return {last} : {out_t} }}")
    return "\n".join(L)


def rope_call(shape=(2, 3, 16, 32), freq_cols=32, dtype="f32"):
    """custom_call @fused_rope: x [.., S, D], frequencies [S, D] (cos | sin) or [S, D / 2] (angles)."""
    t = "x".join(map(str, shape)) + "x" + dtype
    f = f"{shape[-2]}x{freq_cols}x{dtype}"
    return f"""func.func @main(%x: tensor<{t}>, %f: tensor<{f}>) -> tensor<{t}> {{
  %r = stablehlo.custom_call @fused_rope(%x, %f) {{backend_config = "{{}}"}} : (tensor<{t}>, tensor<{f}>) -> tensor<{t}>
  return %r : tensor<{t}> }}"""


def elementwise_call(ops, n_inputs, shape=(6, 40), dtype="f32", key="ops", scalar_inputs=()):
    """custom_call @fused_elementwise with the operation list under `key`; inputs listed in
    `scalar_inputs` are rank-0 tensors."""
    t = "x".join(map(str, shape)) + "x" + dtype
    types = [f"tensor<{dtype}>" if i in scalar_inputs else f"tensor<{t}>" for i in range(n_inputs)]
    args = ", ".join(f"%a{i}: {ty}" for i, ty in enumerate(types))
    names = ", ".join(f"%a{i}" for i in range(n_inputs))
    cfg = '{\\"' + key + '\\": [' + ", ".join('\\"' + o + '\\"' for o in ops) + "]}"
    return f"""func.func @main({args}) -> tensor<{t}> {{
  %r = stablehlo.custom_call @fused_elementwise({names}) {{backend_config = "{cfg}"}} : ({", ".join(types)}) -> tensor<{t}>
  return %r : tensor<{t}> }}"""


def batch_norm_call(shape=(2, 5, 5, 16), dtype="f32", eps=1e-5, n_operands=5):
    """custom_call @fused_batch_norm: x [.., C], gamma, beta, mean, variance [C]."""
    t = "x".join(map(str, shape)) + "x" + dtype
    c = f"{shape[-1]}x{dtype}"
    names = ["%x", "%g", "%b", "%m", "%v"][:n_operands]
    types = [f"tensor<{t}>"] + [f"tensor<{c}>"] * (n_operands - 1)
    return f"""func.func @main(%x: tensor<{t}>, %g: tensor<{c}>, %b: tensor<{c}>, %m: tensor<{c}>, %v: tensor<{c}>) -> tensor<{t}> {{
  %r = stablehlo.custom_call @fused_batch_norm({", ".join(names)}) {{backend_config = "{{\\"eps\\": {eps}}}"}} : ({", ".join(types)}) -> tensor<{t}>
  return %r : tensor<{t}> }}"""


def depth_attention_call(lead=(4,), depth=8, hidden=32, dtype="f32", scale=None, query_row=True):
    """custom_call @fused_depth_attention: query [.., 1, H] (or [.., H]), keys and values [.., depth, H]."""
    q = "x".join(map(str, lead + ((1, hidden) if query_row else (hidden,)))) + "x" + dtype
    kv = "x".join(map(str, lead + (depth, hidden))) + "x" + dtype
    cfg = "{}" if scale is None else '{\\"scale\\": ' + repr(float(scale)) + "}"
    return f"""func.func @main(%q: tensor<{q}>, %k: tensor<{kv}>, %v: tensor<{kv}>) -> tensor<{q}> {{
  %r = stablehlo.custom_call @fused_depth_attention(%q, %k, %v) {{backend_config = "{cfg}"}} : (tensor<{q}>, tensor<{kv}>, tensor<{kv}>) -> tensor<{q}>
  return %r : tensor<{q}> }}"""
