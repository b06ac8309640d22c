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


def transformer_block(B=2, S=64, H=4, D=32, F=256, dtype="f32"):
    """One pre-LayerNorm GPT-2 block written out in plain StableHLO (no custom calls), the way a
    tracing front end emits it: LN -> QKV projection -> head split -> causal attention (scores,
    scale, additive mask from iota / compare / select, softmax, PV) -> head merge -> projection
    -> residual -> LN -> FFN with tanh GELU -> residual.
    Arguments: x [B,S,d], ln1 g/b [d], wqkv [d,3d], bqkv [3d], wo [d,d], bo [d], ln2 g/b [d],
    w1 [d,F], b1 [F], w2 [F,d], b2 [d]."""
    d = H * D
    e = dtype
    x3, x2 = f"tensor<{B}x{S}x{d}x{e}>", f"tensor<{B}x{S}x{e}>"
    hd, hs = f"tensor<{B}x{S}x{H}x{D}x{e}>", f"tensor<{B}x{H}x{S}x{D}x{e}>"
    sc, sr = f"tensor<{B}x{H}x{S}x{S}x{e}>", f"tensor<{B}x{H}x{S}x{e}>"
    neg = {"f32": "0xFF800000", "bf16": "0xFF80", "f16": "0xFC00"}[dtype]
    L = []
    emit = L.append

    def layer_norm(tag, src, g, b):
        emit(f"  %{tag}n = stablehlo.constant dense<{float(d)!r}> : {x2}")
        emit(f"  %{tag}eps = stablehlo.constant dense<1.0e-5> : {x2}")
        emit(f"  %{tag}s = stablehlo.reduce({src} init: %zero) applies stablehlo.add across dimensions = [2] : ({x3}, tensor<{e}>) -> {x2}")
        emit(f"  %{tag}mean = stablehlo.divide %{tag}s, %{tag}n : {x2}")
        emit(f"  %{tag}mb = stablehlo.broadcast_in_dim %{tag}mean, dims = [0, 1] : ({x2}) -> {x3}")
        emit(f"  %{tag}c = stablehlo.subtract {src}, %{tag}mb : {x3}")
        emit(f"  %{tag}sq = stablehlo.multiply %{tag}c, %{tag}c : {x3}")
        emit(f"  %{tag}s2 = stablehlo.reduce(%{tag}sq init: %zero) applies stablehlo.add across dimensions = [2] : ({x3}, tensor<{e}>) -> {x2}")
        emit(f"  %{tag}var = stablehlo.divide %{tag}s2, %{tag}n : {x2}")
        emit(f"  %{tag}ve = stablehlo.add %{tag}var, %{tag}eps : {x2}")
        emit(f"  %{tag}r = stablehlo.rsqrt %{tag}ve : {x2}")
        emit(f"  %{tag}rb = stablehlo.broadcast_in_dim %{tag}r, dims = [0, 1] : ({x2}) -> {x3}")
        emit(f"  %{tag}xn = stablehlo.multiply %{tag}c, %{tag}rb : {x3}")
        emit(f"  %{tag}gb = stablehlo.broadcast_in_dim {g}, dims = [2] : (tensor<{d}x{e}>) -> {x3}")
        emit(f"  %{tag}bb = stablehlo.broadcast_in_dim {b}, dims = [2] : (tensor<{d}x{e}>) -> {x3}")
        emit(f"  %{tag}y = stablehlo.multiply %{tag}xn, %{tag}gb : {x3}")
        emit(f"  %{tag}o = stablehlo.add %{tag}y, %{tag}bb : {x3}")
        return f"%{tag}o"

    def linear(tag, src, w, b, n_in, n_out):
        ti, to = f"tensor<{B}x{S}x{n_in}x{e}>", f"tensor<{B}x{S}x{n_out}x{e}>"
        emit(f"  %{tag}d = stablehlo.dot_general {src}, {w}, contracting_dims = [2] x [0] : ({ti}, tensor<{n_in}x{n_out}x{e}>) -> {to}")
        emit(f"  %{tag}bb = stablehlo.broadcast_in_dim {b}, dims = [2] : (tensor<{n_out}x{e}>) -> {to}")
        emit(f"  %{tag}o = stablehlo.add %{tag}d, %{tag}bb : {to}")
        return f"%{tag}o"

    args = (f"%x: {x3}, %g1: tensor<{d}x{e}>, %b1: tensor<{d}x{e}>, %wqkv: tensor<{d}x{3 * d}x{e}>, %bqkv: tensor<{3 * d}x{e}>, "
            f"%wo: tensor<{d}x{d}x{e}>, %bo: tensor<{d}x{e}>, %g2: tensor<{d}x{e}>, %b2: tensor<{d}x{e}>, "
            f"%w1: tensor<{d}x{F}x{e}>, %c1: tensor<{F}x{e}>, %w2: tensor<{F}x{d}x{e}>, %c2: tensor<{d}x{e}>")
    emit(f"func.func @main({args}) -> {x3} {{")
    emit(f"  %zero = stablehlo.constant dense<0.0> : tensor<{e}>")
    h = layer_norm("ln1", "%x", "%g1", "%b1")
    qkv = linear("qkv", h, "%wqkv", "%bqkv", d, 3 * d)
    for i, name in enumerate("qkv"):
        emit(f"  %{name}s = stablehlo.slice {qkv} [0:{B}, 0:{S}, {i * d}:{(i + 1) * d}] : (tensor<{B}x{S}x{3 * d}x{e}>) -> {x3}")
        emit(f"  %{name}r = stablehlo.reshape %{name}s : ({x3}) -> {hd}")
        emit(f"  %{name}h = stablehlo.transpose %{name}r, dims = [0, 2, 1, 3] : ({hd}) -> {hs}")
    emit(f"  %s0 = stablehlo.dot_general %qh, %kh, batching_dims = [0, 1] x [0, 1], contracting_dims = [3] x [3] : ({hs}, {hs}) -> {sc}")
    emit(f"  %scale = stablehlo.constant dense<{D ** -0.5!r}> : {sc}")
    emit(f"  %s1 = stablehlo.multiply %s0, %scale : {sc}")
    # additive causal mask [S, S]: 0 where key <= query, -inf elsewhere
    emit(f"  %qi = stablehlo.iota dim = 0 : tensor<{S}x{S}xi32>")
    emit(f"  %ki = stablehlo.iota dim = 1 : tensor<{S}x{S}xi32>")
    emit(f"  %keep = stablehlo.compare LE, %ki, %qi, SIGNED : (tensor<{S}x{S}xi32>, tensor<{S}x{S}xi32>) -> tensor<{S}x{S}xi1>")
    emit(f"  %mz = stablehlo.constant dense<0.0> : tensor<{S}x{S}x{e}>")
    emit(f"  %mn = stablehlo.constant dense<{neg}> : tensor<{S}x{S}x{e}>")
    emit(f"  %mask = stablehlo.select %keep, %mz, %mn : tensor<{S}x{S}xi1>, tensor<{S}x{S}x{e}>")
    emit(f"  %mbc = stablehlo.broadcast_in_dim %mask, dims = [2, 3] : (tensor<{S}x{S}x{e}>) -> {sc}")
    emit(f"  %s2 = stablehlo.add %s1, %mbc : {sc}")
    emit(f"  %ninf = stablehlo.constant dense<{neg}> : tensor<{e}>")
    emit(f"  %m = stablehlo.reduce(%s2 init: %ninf) applies stablehlo.maximum across dimensions = [3] : ({sc}, tensor<{e}>) -> {sr}")
    emit(f"  %mb = stablehlo.broadcast_in_dim %m, dims = [0, 1, 2] : ({sr}) -> {sc}")
    emit(f"  %sh = stablehlo.subtract %s2, %mb : {sc}")
    emit(f"  %ex = stablehlo.exponential %sh : {sc}")
    emit(f"  %es = stablehlo.reduce(%ex init: %zero) applies stablehlo.add across dimensions = [3] : ({sc}, tensor<{e}>) -> {sr}")
    emit(f"  %esb = stablehlo.broadcast_in_dim %es, dims = [0, 1, 2] : ({sr}) -> {sc}")
    emit(f"  %p = stablehlo.divide %ex, %esb : {sc}")
    emit(f"  %oh = stablehlo.dot_general %p, %vh, batching_dims = [0, 1] x [0, 1], contracting_dims = [3] x [2] : ({sc}, {hs}) -> {hs}")
    emit(f"  %ot = stablehlo.transpose %oh, dims = [0, 2, 1, 3] : ({hs}) -> {hd}")
    emit(f"  %om = stablehlo.reshape %ot : ({hd}) -> {x3}")
    proj = linear("proj", "%om", "%wo", "%bo", d, d)
    emit(f"  %res1 = stablehlo.add %x, {proj} : {x3}")
    h2 = layer_norm("ln2", "%res1", "%g2", "%b2")
    up = linear("up", h2, "%w1", "%c1", d, F)
    tf = f"tensor<{B}x{S}x{F}x{e}>"
    for name, val in (("half", 0.5), ("one", 1.0), ("coeff", 0.044715), ("kk", 0.7978845608)):
        emit(f"  %{name} = stablehlo.constant dense<{val!r}> : {tf}")
    emit(f"  %u2 = stablehlo.multiply {up}, {up} : {tf}")
    emit(f"  %u3 = stablehlo.multiply %u2, {up} : {tf}")
    emit(f"  %cu3 = stablehlo.multiply %coeff, %u3 : {tf}")
    emit(f"  %inner = stablehlo.add {up}, %cu3 : {tf}")
    emit(f"  %targ = stablehlo.multiply %kk, %inner : {tf}")
    emit(f"  %th = stablehlo.tanh %targ : {tf}")
    emit(f"  %opt = stablehlo.add %one, %th : {tf}")
    emit(f"  %hu = stablehlo.multiply %half, {up} : {tf}")
    emit(f"  %act = stablehlo.multiply %hu, %opt : {tf}")
    down = linear("down", "%act", "%w2", "%c2", F, d)
    emit(f"  %res2 = stablehlo.add %res1, {down} : {x3}")
    emit(f"  return %res2 : {x3} }}")
    return "\n".join(L)


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


GPT2_LAYER_PARAMS = ["ln1_g", "ln1_b", "w_qkv", "b_qkv", "w_o", "b_o", "ln2_g", "ln2_b", "w_fc", "b_fc", "w_proj", "b_proj"]


def gpt2_program(B, S, n_layer, H, D, F, vocab, n_pos, dtype="bf16"):
    """A whole pre-LayerNorm GPT-2 forward in plain StableHLO with fp32 parameters converted to the
    compute type where they are used: token gather + learned positions, `n_layer` blocks as
    transformer_block writes them, final LayerNorm, logits against the tied embedding.
    Arguments: ids [B,S] i32, wte [vocab,d], wpe [n_pos,d], then per layer the twelve tensors of
    GPT2_LAYER_PARAMS, then lnf_g, lnf_b (all f32).  Result: logits [B,S,vocab] in `dtype`."""
    import re
    d, e = H * D, dtype
    x3, x3f = f"tensor<{B}x{S}x{d}x{e}>", f"tensor<{B}x{S}x{d}xf32>"
    shapes = {"ln1_g": [d], "ln1_b": [d], "w_qkv": [d, 3 * d], "b_qkv": [3 * d], "w_o": [d, d], "b_o": [d], "ln2_g": [d], "ln2_b": [d],
              "w_fc": [d, F], "b_fc": [F], "w_proj": [F, d], "b_proj": [d]}
    tt = lambda shape, et: "tensor<" + "".join(f"{n}x" for n in shape) + et + ">"
    args = [f"%ids: tensor<{B}x{S}xi32>", f"%wte: {tt([vocab, d], 'f32')}", f"%wpe: {tt([n_pos, d], 'f32')}"]
    for i in range(n_layer):
        args += [f"%p{i}_{n}: {tt(shapes[n], 'f32')}" for n in GPT2_LAYER_PARAMS]
    args += [f"%lnf_g: {tt([d], 'f32')}", f"%lnf_b: {tt([d], 'f32')}"]
    out_t = tt([B, S, vocab], e)
    L = [f"func.func @main({', '.join(args)}) -> {out_t} {{", f"  %zero = stablehlo.constant dense<0.0> : tensor<{e}>"]
    L.append(f'  %tok = "stablehlo.gather"(%wte, %ids) {{ dimension_numbers = #stablehlo.gather<offset_dims = [2], collapsed_slice_dims = [0], '
             f'start_index_map = [0], index_vector_dim = 2>, slice_sizes = array<i64: 1, {d}>, indices_are_sorted = false }} '
             f': ({tt([vocab, d], "f32")}, tensor<{B}x{S}xi32>) -> {x3f}')
    L.append(f"  %pos = stablehlo.slice %wpe [0:{S}, 0:{d}] : ({tt([n_pos, d], 'f32')}) -> {tt([S, d], 'f32')}")
    L.append(f"  %posb = stablehlo.broadcast_in_dim %pos, dims = [1, 2] : ({tt([S, d], 'f32')}) -> {x3f}")
    L.append(f"  %emb = stablehlo.add %tok, %posb : {x3f}")
    L.append(f"  %h0 = stablehlo.convert %emb : ({x3f}) -> {x3}")
    block = transformer_block(B, S, H, D, F, e).split("\n")[2:-1]          # without the signature, %zero and the return
    arg_of = dict(zip(["g1", "b1", "wqkv", "bqkv", "wo", "bo", "g2", "b2", "w1", "c1", "w2", "c2"], GPT2_LAYER_PARAMS))
    cur = "%h0"
    for i in range(n_layer):
        for n in GPT2_LAYER_PARAMS:
            L.append(f"  %c{i}_{n} = stablehlo.convert %p{i}_{n} : ({tt(shapes[n], 'f32')}) -> {tt(shapes[n], e)}")

        def rename(m, i=i, cur=cur):
            name = m.group(1)
            if name == "zero":
                return "%zero"
            if name == "x":
                return cur
            if name in arg_of:
                return f"%c{i}_{arg_of[name]}"
            return f"%L{i}_{name}"
        L += [re.sub(r"%([A-Za-z0-9_]+)", rename, ln) for ln in block]
        cur = f"%L{i}_res2"
    # final LayerNorm: the block's own spelling, on the last residual stream
    ln = transformer_block(B, S, H, D, F, e).split("\n")[2:19]
    L.append(f"  %cf_g = stablehlo.convert %lnf_g : ({tt([d], 'f32')}) -> {tt([d], e)}")
    L.append(f"  %cf_b = stablehlo.convert %lnf_b : ({tt([d], 'f32')}) -> {tt([d], e)}")
    final = {"x": cur, "g1": "%cf_g", "b1": "%cf_b", "zero": "%zero"}
    L += [re.sub(r"%([A-Za-z0-9_]+)", lambda m: final.get(m.group(1), f"%F_{m.group(1)}"), l2) for l2 in ln]
    L.append(f"  %cwte = stablehlo.convert %wte : ({tt([vocab, d], 'f32')}) -> {tt([vocab, d], e)}")
    L.append(f"  %logits = stablehlo.dot_general %F_ln1o, %cwte, contracting_dims = [2] x [1] : ({x3}, {tt([vocab, d], e)}) -> {out_t}")
    L.append(f"  return %logits : {out_t} }}")
    return "\n".join(L)
