"""StableHLO programs written the way a tracing front end emits them (no custom calls):
one pre-LayerNorm transformer block and a whole GPT-2 forward.  Used by the tests of the
pattern recogniser and by the benchmark's from-text GPT-2 workload; the reference builds
its benchmark programs the same way, from text templates
(Sources/MetalHLOBenchmarks/ModelBenchmarks.swift:1083-1115)."""

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
