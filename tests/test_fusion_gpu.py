"""GPU: modules compiled with pattern recognition (the default) and as written (O0) agree
with each other and with the float64 oracle; fp32 tolerance 1e-5, bf16 2e-2, with the
floor max(tol, tol*|e|)."""
import numpy as np
import pytest

from oracle import oracle
from tests import fusion_modules as M

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def sess():
    from metalhlo_amd import capi
    s = capi.Session()
    yield s
    s.close()


def close(got, exp, tol):
    exp = np.asarray(exp, dtype=np.float64)
    got = np.asarray(got, dtype=np.float64)
    assert got.shape == exp.shape
    assert np.all(np.abs(got - exp) <= np.maximum(tol, tol * np.abs(exp))), np.abs(got - exp).max()


def both(sess, text, inputs, expect_op):
    fused, plain = sess.compile(text), sess.compile(text, 0)
    assert expect_op in sess.ops(fused) and expect_op not in sess.ops(plain)
    (a,), (b,) = sess.run(fused, inputs), sess.run(plain, inputs)
    sess.lib.mhlo_executable_destroy(fused)
    sess.lib.mhlo_executable_destroy(plain)
    return a, b


def test_softmax_gelu_norms(sess):
    rng = np.random.default_rng(81)
    x = rng.standard_normal((8, 32)).astype(np.float32)
    a, b = both(sess, M.SOFTMAX, [(x, "f32")], "fused_softmax")
    close(a, oracle.softmax(x.astype(np.float64)), 1e-5)
    close(b, oracle.softmax(x.astype(np.float64)), 1e-5)
    a, b = both(sess, M.SOFTMAX_AXIS0, [(x, "f32")], "fused_softmax")
    close(a, oracle.softmax(x.astype(np.float64), axis=0), 1e-5)
    close(b, a, 1e-5)
    x = rng.uniform(-4, 4, (4, 64)).astype(np.float32)
    a, b = both(sess, M.GELU, [(x, "f32")], "fused_gelu")
    close(a, oracle.gelu_tanh(x.astype(np.float64)), 1e-5)
    close(b, oracle.gelu_tanh(x.astype(np.float64)), 1e-5)
    x = (3 + 2 * rng.standard_normal((16, 64))).astype(np.float32)
    g = (1 + 0.1 * rng.standard_normal(64)).astype(np.float32)
    bt = (0.1 * rng.standard_normal(64)).astype(np.float32)
    a, b = both(sess, M.LAYER_NORM, [(x, "f32"), (g, "f32"), (bt, "f32")], "fused_layer_norm")
    exp = oracle.layer_norm(x.astype(np.float64), g.astype(np.float64), bt.astype(np.float64), 1e-5)
    close(a, exp, 1e-5)
    close(b, exp, 2e-5)      # the decomposed form subtracts the mean in fp32 before squaring
    a, b = both(sess, M.RMS_NORM, [(x, "f32"), (g, "f32")], "fused_rms_norm")
    exp = oracle.rms_norm(x.astype(np.float64), g.astype(np.float64), 1e-6)
    close(a, exp, 1e-5)
    close(b, exp, 1e-5)


@pytest.mark.parametrize("form", ["le", "ge_swapped", "gt_drop", "big_negative", "anti", "keep_one"])
def test_masks_built_from_iotas(sess, form):
    """Causal spellings run with the causal flag, the others with their mask: both must equal the
    oracle with the mask the program describes, and the program run as written."""
    B, H, S, D = 2, 2, 64, 32
    rng = np.random.default_rng(83)
    q, k, v = (rng.standard_normal((B, H, S, D)).astype(np.float32) for _ in range(3))
    qi, ki = np.arange(S)[:, None], np.arange(S)[None, :]
    keep = (ki >= qi) if form == "anti" else (ki <= qi)
    mask = np.where(keep, 1.0 if form == "keep_one" else 0.0, -1e30 if form == "big_negative" else -np.inf)
    exp = oracle.attention(q.astype(np.float64), k.astype(np.float64), v.astype(np.float64), scale=D ** -0.5, mask=mask)
    a, b = both(sess, M.masked_attention(form), [(q, "f32"), (k, "f32"), (v, "f32")], "fused_scaled_dot_product_attention")
    close(a, exp, 1e-5)
    close(b, exp, 1e-5)


def test_keepdims_forms(sess):
    rng = np.random.default_rng(82)
    x = rng.standard_normal((8, 32)).astype(np.float32)
    a, b = both(sess, M.SOFTMAX_KEEPDIMS, [(x, "f32")], "fused_softmax")
    close(a, oracle.softmax(x.astype(np.float64)), 1e-5)
    close(b, oracle.softmax(x.astype(np.float64)), 1e-5)
    x = (3 + 2 * rng.standard_normal((16, 64))).astype(np.float32)
    g = (1 + 0.1 * rng.standard_normal(64)).astype(np.float32)
    bt = (0.1 * rng.standard_normal(64)).astype(np.float32)
    a, b = both(sess, M.LAYER_NORM_KEEPDIMS, [(x, "f32"), (g, "f32"), (bt, "f32")], "fused_layer_norm")
    exp = oracle.layer_norm(x.astype(np.float64), g.astype(np.float64), bt.astype(np.float64), 1e-5)
    close(a, exp, 1e-5)
    close(b, exp, 2e-5)
    # the look-alike that spreads the row statistic over axis 0 runs as written: out[i, j] = e[i, j] / sum_k e[j, k]
    x = rng.standard_normal((8, 8)).astype(np.float32)
    exe = sess.compile(M.NOT_SOFTMAX_WRONG_SPREAD)
    (got,) = sess.run(exe, [(x, "f32")])
    sess.lib.mhlo_executable_destroy(exe)
    x64 = x.astype(np.float64)
    e = np.exp(x64 - x64.max(axis=1)[None, :])
    close(got, e / e.sum(axis=1)[None, :], 1e-5)


@pytest.mark.parametrize("with_mask,transpose_k,divide", [(False, True, False), (True, False, True), (True, True, False)])
def test_attention_chain(sess, with_mask, transpose_k, divide):
    B, H, S, D = 2, 3, 64, 32
    rng = np.random.default_rng(82)
    q, k, v = (rng.standard_normal((B, H, S, D)).astype(np.float32) for _ in range(3))
    inputs = [(q, "f32"), (k, "f32"), (v, "f32")]
    mask = None
    if with_mask:
        mask = np.where(np.arange(S)[None, :] > np.arange(S)[:, None], -np.inf, 0.0).astype(np.float32)
        inputs.append((mask, "f32"))
    text = M.attention(B, H, S, D, with_mask=with_mask, transpose_k=transpose_k, divide=divide)
    a, b = both(sess, text, inputs, "fused_scaled_dot_product_attention")
    exp = oracle.attention(q, k, v, scale=D ** -0.5, mask=mask)
    close(a, exp, 1e-5)
    close(b, exp, 1e-5)


def test_attention_chain_bf16(sess):
    B, H, S, D = 1, 4, 128, 64
    rng = np.random.default_rng(83)
    bits = [oracle.bf16_round_bits(rng.standard_normal((B, H, S, D)).astype(np.float32)) for _ in range(3)]
    text = M.attention(B, H, S, D, dtype="bf16")
    fused = sess.compile(text)
    assert sess.ops(fused) == ["fused_scaled_dot_product_attention"]
    (o,) = sess.run(fused, [(x, "bf16") for x in bits])
    q, k, v = (oracle.bf16_bits_to_f32(x).astype(np.float64) for x in bits)
    close(oracle.bf16_bits_to_f32(o), oracle.attention(q, k, v, scale=D ** -0.5), 2e-2)


def test_matmul_bias_activation(sess):
    rng = np.random.default_rng(84)
    x = rng.uniform(-1, 1, (32, 64)).astype(np.float32)
    w = rng.uniform(-1, 1, (64, 128)).astype(np.float32)
    bias = rng.standard_normal(128).astype(np.float32)
    ins = [(x, "f32"), (w, "f32"), (bias, "f32")]
    a, b = both(sess, M.FFN_UP, ins, "fused_matmul_bias_activation")
    exp = oracle.matmul_bias_act(x.astype(np.float64), w.astype(np.float64), bias.astype(np.float64), "gelu")
    close(a, exp, 1e-5)
    close(b, exp, 1e-5)
    a, b = both(sess, M.MATMUL_BIAS_RELU, ins, "fused_matmul_bias_activation")
    exp = oracle.matmul_bias_act(x.astype(np.float64), w.astype(np.float64), bias.astype(np.float64), "relu")
    close(a, exp, 1e-5)
    close(b, exp, 1e-5)


def test_erf_gelu_one_pass_layer_norm_and_calls(sess):
    rng = np.random.default_rng(84)
    x = rng.uniform(-4, 4, (4, 64)).astype(np.float32)
    for text in (M.GELU_ERF, M.GELU_ERF_MUL):
        a, b = both(sess, text, [(x, "f32")], "fused_gelu")
        close(a, oracle.gelu_erf(x.astype(np.float64)), 1e-5)
        close(b, oracle.gelu_erf(x.astype(np.float64)), 1e-5)
    # the exact form is not the tanh approximation: the two differ by more than the tolerance somewhere
    assert np.max(np.abs(oracle.gelu_erf(x.astype(np.float64)) - oracle.gelu_tanh(x.astype(np.float64)))) > 1e-4
    x = (3 + 2 * rng.standard_normal((16, 64))).astype(np.float32)
    g = (1 + 0.1 * rng.standard_normal(64)).astype(np.float32)
    bt = (0.1 * rng.standard_normal(64)).astype(np.float32)
    a, b = both(sess, M.LAYER_NORM_ONE_PASS, [(x, "f32"), (g, "f32"), (bt, "f32")], "fused_layer_norm")
    exp = oracle.layer_norm(x.astype(np.float64), g.astype(np.float64), bt.astype(np.float64), 1e-5)
    close(a, exp, 1e-5)
    close(b, exp, 1e-4)      # as written: mean(x^2) - mean(x)^2 in fp32 cancels (mean 3, deviation 2)
    # calls: the flat program equals its own restatement
    x = rng.standard_normal((8, 16)).astype(np.float32)
    y = rng.standard_normal((8, 16)).astype(np.float32)
    exe = sess.compile(M.CALLS)
    t, u = sess.run(exe, [(x, "f32"), (y, "f32")])
    sess.lib.mhlo_executable_destroy(exe)
    s = x + y
    r0, r1 = np.where(s > 0, s, 0), -s
    assert np.array_equal(t, r0 * r1) and np.array_equal(u, np.where(r1 < 0, r1, r0 * r1))


@pytest.mark.parametrize("act", ["gelu", "gelu_exact", "relu", "silu", "mish"])
def test_fused_ffn(sess, act):
    """("mish": a name the reference's handler does not know, which there and here means no
    activation, CustomCallHandlers.swift:905.  "gelu_exact" is the erf form: this build's choice, the
    reference computes the tanh form under that name; the expectation is not pinned by the reference.)"""
    rng = np.random.default_rng(85)
    x = rng.standard_normal((4, 32, 64)).astype(np.float32)
    up = (0.2 * rng.standard_normal((64, 256))).astype(np.float32)
    down = (0.2 * rng.standard_normal((256, 64))).astype(np.float32)
    exe = sess.compile(M.FFN_CUSTOM_CALL.replace("ACT", act))
    (got,) = sess.run(exe, [(x, "f32"), (up, "f32"), (down, "f32")])
    sess.lib.mhlo_executable_destroy(exe)
    h = oracle.ACTIVATIONS.get(act, oracle.ACTIVATIONS["none"])(oracle.gemm(x.astype(np.float64).reshape(-1, 64), up.astype(np.float64)))
    close(got, oracle.gemm(h, down.astype(np.float64)).reshape(x.shape), 2e-5)


@pytest.mark.parametrize("dtype,first,d", [("bf16", 0, 64), ("bf16", 5, 48), ("f32", 3, 64), ("f16", 0, 30)])
def test_token_embedding(sess, dtype, first, d):
    """The embedding head as one kernel and as written give the same bits (one fp32 sum, one
    rounding), ids outside the table clamped as gather clamps them; both equal
    table[ids] + positions[first + s] rounded to the result type."""
    B, S, vocab, n_pos = 3, 16, 50, 24
    rng = np.random.default_rng(97)
    ids = rng.integers(0, vocab, (B, S)).astype(np.int32)
    ids[0, 0], ids[1, 3], ids[2, 15] = -7, vocab, vocab + 1000
    wte = rng.standard_normal((vocab, d)).astype(np.float32)
    wpe = rng.standard_normal((n_pos, d)).astype(np.float32)
    text = M.embedding(B, S, d, vocab, n_pos, dtype, first)
    a, b = both(sess, text, [(ids, "i32"), (wte, "f32"), (wpe, "f32")], "fused_token_embedding")
    assert np.array_equal(a, b)
    exp = wte[np.clip(ids, 0, vocab - 1)] + wpe[None, first:first + S]          # fp32 sum
    if dtype == "bf16":
        assert np.array_equal(a, oracle.bf16_round_bits(exp))
    else:
        assert np.array_equal(np.asarray(a, dtype=np.float32), exp.astype({"f32": np.float32, "f16": np.float16}[dtype]).astype(np.float32))


def _to(a, dtype):
    """numpy float -> (array, element type name) as Session.run takes it, rounded to `dtype`."""
    if dtype == "f32":
        return np.asarray(a, np.float32), "f32"
    if dtype == "bf16":
        return oracle.bf16_round_bits(np.asarray(a, np.float32)).reshape(np.shape(a)), "bf16"
    return np.asarray(a, np.float16), "f16"


def _from(a, dtype):
    return oracle.bf16_bits_to_f32(a).astype(np.float64) if dtype == "bf16" else np.asarray(a, np.float64)


@pytest.mark.parametrize("dtype", ["f32", "bf16", "f16"])
@pytest.mark.parametrize("shape,table", [((2, 3, 16, 32), True), ((2, 3, 16, 32), False), ((1, 5, 9, 6), False), ((24, 128), True),
                                         ((4, 2, 33, 64), False)],
                         ids=["table", "angles", "odd-half", "rank2", "ragged-seq"])
def test_fused_rope(sess, shape, table, dtype):
    """Rotary position embedding through the C API against the oracle: cos | sin table and angle
    forms, half widths that are no whole 16-byte vectors, every element type."""
    rng = np.random.default_rng(91)
    S, D = shape[-2], shape[-1]
    x = rng.standard_normal(shape)
    th = rng.uniform(-3, 3, (S, D // 2))
    f = np.concatenate([np.cos(th), np.sin(th)], -1) if table else th
    (xa, _), (fa, _) = _to(x, dtype), _to(f, dtype)
    exe = sess.compile(M.rope_call(shape, f.shape[-1], dtype))
    (got,) = sess.run(exe, [(xa, dtype), (fa, dtype)])
    sess.lib.mhlo_executable_destroy(exe)
    exp = oracle.rope(_from(xa, dtype), _from(fa, dtype))
    close(_from(got, dtype), exp, 1e-5 if dtype == "f32" else 2e-2)
    if dtype == "f32":       # a rotation: every pair keeps its norm
        g = np.asarray(got, np.float64)
        h = D // 2
        assert np.allclose(g[..., :h] ** 2 + g[..., h:] ** 2, x[..., :h].astype(np.float32).astype(np.float64) ** 2 +
                           x[..., h:].astype(np.float32).astype(np.float64) ** 2, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("dtype", ["f32", "bf16", "f16"])
@pytest.mark.parametrize("ops,n_in,scalars,shape", [
    (["add", "multiply"], 3, (), (6, 40)),                       # the reference's example
    (["tanh", "add", "negate", "abs"], 2, (), (6, 40)),
    (["multiply", "exponential", "logistic"], 2, (1,), (6, 40)),   # a rank-0 right operand
    (["maximum", "minimum", "subtract", "divide"], 5, (), (3, 7)),  # no whole vectors: the scalar form
    (["abs", "sqrt", "rsqrt", "log"], 1, (), (5, 8)),
    (["sine", "cosine", "floor", "ceil"], 1, (), (4, 16)),
], ids=["add-mul", "unary-mix", "scalar-rhs", "five-inputs", "roots", "trig-round"])
def test_fused_elementwise(sess, ops, n_in, scalars, shape, dtype):
    """Elementwise chains in one launch against the oracle (fp32 chain, one rounding at the store;
    the bf16 / f16 bar is the per-operator 2e-2)."""
    rng = np.random.default_rng(93)
    ins = []
    for i in range(n_in):
        a = rng.uniform(0.5, 2.0, () if i in scalars else shape) * (1 if ops[0] in ("abs", "sqrt") or i else rng.choice([-1, 1], shape))
        ins.append(_to(a, dtype))
    text = M.elementwise_call(ops, n_in, shape, dtype, scalar_inputs=scalars)
    exe = sess.compile(text)
    (got,) = sess.run(exe, [(a, t) for a, t in ins])
    sess.lib.mhlo_executable_destroy(exe)
    exp = oracle.elementwise_chain([_from(a, dtype) for a, _ in ins], ops)
    exp = np.broadcast_to(exp, shape)
    g = _from(got, dtype)
    if ops[-1] in ("floor", "ceil"):      # integers: a last-bit difference in front of the rounding may move one
        assert np.mean(g == exp) > 0.98 and np.max(np.abs(g - exp)) <= 1.0
    else:
        close(g, exp, 1e-5 if dtype == "f32" else 2e-2)


def test_trig_and_rounding_operations_of_the_front_end(sess):
    """stablehlo.sine / cosine / floor / ceil as plain operations (they came with fused_elementwise)."""
    text = """func.func @main(%x: tensor<4x8xf32>) -> (tensor<4x8xf32>, tensor<4x8xf32>) {
      %0 = stablehlo.sine %x : tensor<4x8xf32>
      %1 = stablehlo.cosine %x : tensor<4x8xf32>
      %2 = stablehlo.multiply %0, %1 : tensor<4x8xf32>
      %3 = stablehlo.floor %x : tensor<4x8xf32>
      %4 = stablehlo.ceil %x : tensor<4x8xf32>
      %5 = stablehlo.subtract %4, %3 : tensor<4x8xf32>
      return %2, %5 : tensor<4x8xf32>, tensor<4x8xf32> }"""
    x = np.random.default_rng(95).uniform(-4, 4, (4, 8)).astype(np.float32)
    x[0, :3] = [-1.0, 0.0, 2.0]
    exe = sess.compile(text)
    a, b = sess.run(exe, [(x, "f32")])
    sess.lib.mhlo_executable_destroy(exe)
    close(a, np.sin(x.astype(np.float64)) * np.cos(x.astype(np.float64)), 1e-5)
    assert np.array_equal(b, np.ceil(x) - np.floor(x))


@pytest.mark.parametrize("dtype", ["f32", "bf16", "f16"])
@pytest.mark.parametrize("shape", [(2, 5, 5, 16), (64, 30), (3, 7, 129), (4096, 64)], ids=["nhwc", "rank2-odd", "no-vectors", "large"])
def test_fused_batch_norm(sess, shape, dtype):
    """Normalisation with given statistics through the C API against the oracle; with the batch's own
    statistics every channel of the fp32 result has mean beta."""
    rng = np.random.default_rng(95)
    C_ = shape[-1]
    x = rng.standard_normal(shape) * 2 + 0.5
    g, b = rng.uniform(0.5, 1.5, C_), rng.standard_normal(C_)
    flat = x.reshape(-1, C_)
    mu, var = flat.mean(axis=0), flat.var(axis=0)
    arrs = [_to(a, dtype)[0] for a in (x, g, b, mu, var)]
    exe = sess.compile(M.batch_norm_call(shape, dtype, eps=0.001))
    (got,) = sess.run(exe, [(a, dtype) for a in arrs])
    sess.lib.mhlo_executable_destroy(exe)
    exp = oracle.batch_norm(*[_from(a, dtype) for a in arrs], eps=0.001)
    close(_from(got, dtype), exp, 1e-5 if dtype == "f32" else 2e-2)
    if dtype == "f32":
        assert np.allclose(np.asarray(got, np.float64).reshape(-1, C_).mean(axis=0), b, atol=1e-4)


@pytest.mark.parametrize("dtype", ["f32", "bf16", "f16"])
@pytest.mark.parametrize("lead,depth,hidden,row", [((4,), 8, 32, True), ((2, 3), 32, 768, True), ((5,), 1, 40, True),
                                                   ((3,), 64, 257, False), ((1,), 4, 16, True)],
                         ids=["small", "attnres-768", "one-row", "depth64-odd-hidden", "batch1"])
def test_fused_depth_attention(sess, lead, depth, hidden, row, dtype):
    """Attention of one query row over a few stored rows through the C API against the oracle."""
    rng = np.random.default_rng(96)
    q = rng.standard_normal(lead + ((1, hidden) if row else (hidden,)))
    k, v = rng.standard_normal(lead + (depth, hidden)), rng.standard_normal(lead + (depth, hidden))
    scale = hidden ** -0.5
    arrs = [_to(a, dtype)[0] for a in (q, k, v)]
    exe = sess.compile(M.depth_attention_call(lead, depth, hidden, dtype, scale, row))
    (got,) = sess.run(exe, [(a, dtype) for a in arrs])
    sess.lib.mhlo_executable_destroy(exe)
    exp = oracle.depth_attention(*[_from(a, dtype) for a in arrs], scale=scale)
    close(_from(got, dtype), exp, 1e-5 if dtype == "f32" else 2e-2)


def test_fused_depth_attention_reference_cases(sess):
    """The reference's own cases (Tests/MetalHLOCoreTests/DepthAttentionTests.swift:46-137) at its tolerances:
    equal keys give the mean of the value rows (1e-3), one dominant key selects its value row (0.1)."""
    rng = np.random.default_rng(97)
    q = rng.uniform(-1, 1, (1, 1, 8)).astype(np.float32)
    k = np.ones((1, 4, 8), np.float32)
    v = np.arange(32, dtype=np.float32).reshape(1, 4, 8)
    exe = sess.compile(M.depth_attention_call((1,), 4, 8, "f32", 8 ** -0.5))
    (got,) = sess.run(exe, [(q, "f32"), (k, "f32"), (v, "f32")])
    sess.lib.mhlo_executable_destroy(exe)
    assert np.all(np.abs(np.asarray(got).reshape(8) - v.mean(axis=1).reshape(8)) < 1e-3)
    q = np.zeros((1, 1, 16), np.float32); q[0, 0, 0] = 10.0
    k = np.zeros((1, 4, 16), np.float32); k[0, 2, 0] = 10.0
    v = np.zeros((1, 4, 16), np.float32); v[0, 2] = np.arange(1, 17)
    exe = sess.compile(M.depth_attention_call((1,), 4, 16, "f32", 1.0))
    (got,) = sess.run(exe, [(q, "f32"), (k, "f32"), (v, "f32")])
    sess.lib.mhlo_executable_destroy(exe)
    assert np.all(np.abs(np.asarray(got).reshape(16) - np.arange(1, 17)) < 0.1)
