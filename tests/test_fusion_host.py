"""CPU: the pattern recogniser of the C++ host rewrites decomposed subgraphs into the
fused custom calls, and refuses when that would change the program (interior value used
elsewhere, wrong constants).  Checked through the operation list an executable reports."""
import os

import pytest

os.environ.setdefault("METALHLO_ALLOW_NO_DEVICE", "1")
from metalhlo_amd import capi   # noqa: E402
from tests import fusion_modules as M   # noqa: E402


@pytest.fixture(scope="module")
def sess():
    s = capi.Session()
    yield s
    s.close()


def ops(sess, text, level=None):
    exe = sess.compile(text, level)
    try:
        return sess.ops(exe)
    finally:
        sess.lib.mhlo_executable_destroy(exe)


def test_softmax_chain_becomes_one_call(sess):
    assert ops(sess, M.SOFTMAX) == ["fused_softmax"]
    assert ops(sess, M.SOFTMAX_AXIS0) == ["fused_softmax"]
    # O0 runs the module as written
    assert "fused_softmax" not in ops(sess, M.SOFTMAX, 0) and "reduce" in ops(sess, M.SOFTMAX, 0)
    # the exponentials are a result of the function too: nothing may be absorbed
    assert "fused_softmax" not in ops(sess, M.SOFTMAX_ESCAPING)


def test_keepdims_statistics_are_followed(sess):
    """Statistics carried with a unit dim (broadcast_in_dim or reshape to [rows, 1], arithmetic on
    that shape, one spreading broadcast at the end) are the same patterns; a statistic spread
    over the other axis is not."""
    assert ops(sess, M.SOFTMAX_KEEPDIMS) == ["fused_softmax"]
    assert ops(sess, M.LAYER_NORM_KEEPDIMS) == ["fused_layer_norm"]
    assert "fused_softmax" not in ops(sess, M.NOT_SOFTMAX_WRONG_SPREAD)


def test_whole_transformer_block_fuses(sess):
    """A pre-LayerNorm transformer block in plain StableHLO: 93 operations become 18, every
    LayerNorm, GEMM+bias(+GELU) and the attention core one kernel each; the causal mask the
    program builds from iotas becomes the kernel's causal flag and its operations disappear; the
    two residual adds go into the epilogues of the GEMMs in front of them."""
    got = ops(sess, M.transformer_block())
    assert len(ops(sess, M.transformer_block(), 0)) == 93
    assert [o for o in got if o.startswith("fused_")] == [
        "fused_layer_norm", "fused_matmul_bias_activation", "fused_scaled_dot_product_attention", "fused_matmul_bias_activation",
        "fused_layer_norm", "fused_matmul_bias_activation", "fused_matmul_bias_activation"]
    assert len(got) == 18 and not {"reduce", "exponential", "tanh", "rsqrt", "dot_general", "divide", "iota", "select", "add"} & set(got)


def test_attention_reads_views_of_the_projection(sess):
    """16-bit types with D = 64 / 128: the head split and merge around attention are folded into
    strides (seven operations left, one kernel each); f32 or D = 32 keep the glue (the strided entry is 16-bit MFMA only)."""
    got = ops(sess, M.transformer_block(2, 64, 4, 64, 256, "bf16"))
    assert got == ["fused_layer_norm", "fused_matmul_bias_activation", "fused_scaled_dot_product_attention",
                   "fused_matmul_bias_activation", "fused_layer_norm", "fused_matmul_bias_activation",
                   "fused_matmul_bias_activation"]
    assert len(ops(sess, M.transformer_block(2, 64, 4, 64, 256, "f32"))) == 18
    assert len(ops(sess, M.transformer_block(2, 64, 4, 32, 256, "bf16"))) == 18


def test_residual_goes_into_the_gemm_epilogue_only_when_the_product_has_no_other_user(sess):
    t = "tensor<32x128xf32>"
    head = (f"func.func @main(%x: tensor<32x64xf32>, %w: tensor<64x128xf32>, %b: tensor<128xf32>, %r: {t}) -> RESULT {{\n"
            f"  %d = stablehlo.dot_general %x, %w, contracting_dims = [1] x [0] : (tensor<32x64xf32>, tensor<64x128xf32>) -> {t}\n"
            f"  %bb = stablehlo.broadcast_in_dim %b, dims = [1] : (tensor<128xf32>) -> {t}\n"
            f"  %h = stablehlo.add %d, %bb : {t}\n  %y = stablehlo.add %r, %h : {t}\n")
    assert ops(sess, head.replace("RESULT", t) + f"  return %y : {t} }}") == ["fused_matmul_bias_activation"]
    both = head.replace("RESULT", f"({t}, {t})") + f"  return %y, %h : {t}, {t} }}"
    assert ops(sess, both) == ["fused_matmul_bias_activation", "add"]


def test_views_leave_glue_that_has_other_users(sess):
    """The split tensors are also results of the function here: they must still be produced, while
    attention reads the projection in place all the same."""
    text = M.transformer_block(2, 64, 4, 64, 256, "bf16")
    hs = "tensor<2x4x64x64xbf16>"
    text = text.replace(") -> tensor<2x64x256xbf16> {", f") -> (tensor<2x64x256xbf16>, {hs}) {{")
    text = text.replace("return %res2 : tensor<2x64x256xbf16>", f"return %res2, %kh : tensor<2x64x256xbf16>, {hs}")
    got = ops(sess, text)
    assert got.count("transpose") == 1 and got.count("slice") == 1 and got.count("fused_scaled_dot_product_attention") == 1
    assert len(got) == 10


@pytest.mark.parametrize("form,causal", [("le", True), ("ge_swapped", True), ("gt_drop", True), ("big_negative", True),
                                         ("anti", False), ("keep_one", False)])
def test_causal_mask_from_iotas_becomes_the_causal_flag(sess, form, causal):
    """select(compare(iota, iota), 0, -inf) in any of its spellings is the causal flag (no mask
    operand, no mask operations left); the mirrored comparison or a mask that adds something
    where it keeps stays an additive mask."""
    exe = sess.compile(M.masked_attention(form))
    got = sess.ops(exe)
    sess.lib.mhlo_executable_destroy(exe)
    if causal:
        assert got == ["fused_scaled_dot_product_attention"]
    else:
        assert got.count("fused_scaled_dot_product_attention") == 1 and "select" in got and "iota" in got


def test_gelu_only_with_the_right_constants(sess):
    assert ops(sess, M.GELU) == ["fused_gelu"]
    assert "fused_gelu" not in ops(sess, M.NOT_GELU) and "tanh" in ops(sess, M.NOT_GELU)


def test_norms(sess):
    assert ops(sess, M.LAYER_NORM) == ["fused_layer_norm"]
    assert ops(sess, M.RMS_NORM) == ["fused_rms_norm"]
    # a LayerNorm over rows of 64 whose divisor is 63 is something else
    assert "fused_layer_norm" not in ops(sess, M.LAYER_NORM.replace("dense<64.0>", "dense<63.0>"))


@pytest.mark.parametrize("with_mask", [False, True])
@pytest.mark.parametrize("transpose_k", [False, True])
@pytest.mark.parametrize("divide", [False, True])
def test_attention_absorbs_scale_mask_and_transpose(sess, with_mask, transpose_k, divide):
    got = ops(sess, M.attention(with_mask=with_mask, transpose_k=transpose_k, divide=divide))
    want = ["fused_scaled_dot_product_attention"]
    assert got == want, got


def test_matmul_bias_activation(sess):
    assert ops(sess, M.FFN_UP) == ["fused_matmul_bias_activation"]
    assert ops(sess, M.MATMUL_BIAS_RELU) == ["fused_matmul_bias_activation"]


def test_widening_dot_stays_unfused(sess):
    """bf16 x bf16 -> f32 (what preferred_element_type emits) followed by an f32 bias add is not
    what the fused kernel computes (it reads x, w and writes the result in ONE type): the
    module keeps its dot_general, which converts first."""
    text = ("func.func @main(%x: tensor<32x64xbf16>, %w: tensor<64x128xbf16>, %b: tensor<128xf32>) -> tensor<32x128xf32> {\n"
            "  %d = stablehlo.dot_general %x, %w, contracting_dims = [1] x [0] : (tensor<32x64xbf16>, tensor<64x128xbf16>) -> tensor<32x128xf32>\n"
            "  %bb = stablehlo.broadcast_in_dim %b, dims = [1] : (tensor<128xf32>) -> tensor<32x128xf32>\n"
            "  %h = stablehlo.add %d, %bb : tensor<32x128xf32>\n  return %h : tensor<32x128xf32> }")
    assert ops(sess, text) == ["dot_general", "broadcast_in_dim", "add"]
    assert ops(sess, text, 0) == ["dot_general", "broadcast_in_dim", "add"]


def test_gelu_constants_at_the_precision_of_the_element_type(sess):
    """Near misses (0.79 for sqrt(2/pi), 0.049 for 0.044715) are other functions and stay as
    written; bf16 programs spell the constants as their bf16 roundings and still fuse; f64 has no
    fused kernel and must keep compiling at every level."""
    assert "fused_gelu" not in ops(sess, M.GELU.replace("0.7978845608", "0.79"))
    assert "fused_gelu" not in ops(sess, M.GELU.replace("0.044715", "0.049"))
    assert "fused_gelu" not in ops(sess, M.GELU.replace("0.044715", "0.0447"))
    assert ops(sess, M.GELU.replace("0.7978845608", "0.79788456")) == ["fused_gelu"]
    bf = M.GELU.replace("xf32", "xbf16")
    assert ops(sess, bf) == ["fused_gelu"]
    assert "fused_gelu" not in ops(sess, bf.replace("0.7978845608", "0.79"))        # two bf16 steps away
    f64 = M.GELU.replace("xf32", "xf64")
    assert "fused_gelu" not in ops(sess, f64) and "tanh" in ops(sess, f64)
    assert ops(sess, f64) == ops(sess, f64, 0)


BAD_RESULT_TYPES = {
    "dot_general_small_result":
        "func.func @main(%a: tensor<64x128xf32>, %b: tensor<128x256xf32>) -> tensor<8x8xf32> {\n"
        "  %d = stablehlo.dot_general %a, %b, contracting_dims = [1] x [0] : (tensor<64x128xf32>, tensor<128x256xf32>) -> tensor<8x8xf32>\n"
        "  return %d : tensor<8x8xf32> }",
    "reduce_small_result":
        "func.func @main(%a: tensor<64x128xf32>) -> tensor<4xf32> {\n"
        "  %z = stablehlo.constant dense<0.0> : tensor<f32>\n"
        "  %r = stablehlo.reduce(%a init: %z) applies stablehlo.add across dimensions = [1] : (tensor<64x128xf32>, tensor<f32>) -> tensor<4xf32>\n"
        "  return %r : tensor<4xf32> }",
    "gelu_half_result":
        "func.func @main(%a: tensor<64x128xf32>) -> tensor<32x128xf32> {\n"
        "  %r = stablehlo.custom_call @fused_gelu(%a) : (tensor<64x128xf32>) -> tensor<32x128xf32>\n"
        "  return %r : tensor<32x128xf32> }",
    "softmax_changes_type":
        "func.func @main(%a: tensor<64x128xbf16>) -> tensor<64x128xf32> {\n"
        "  %r = stablehlo.custom_call @fused_softmax(%a) {backend_config = \"{\\\"axis\\\": -1}\"} : (tensor<64x128xbf16>) -> tensor<64x128xf32>\n"
        "  return %r : tensor<64x128xf32> }",
    "matmul_changes_type":
        "func.func @main(%a: tensor<64x128xbf16>, %w: tensor<128x32xbf16>) -> tensor<64x32xf32> {\n"
        "  %r = stablehlo.custom_call @fused_matmul_bias_activation(%a, %w) : (tensor<64x128xbf16>, tensor<128x32xbf16>) -> tensor<64x32xf32>\n"
        "  return %r : tensor<64x32xf32> }",
    "matmul_wrong_shape":
        "func.func @main(%a: tensor<64x128xf32>, %w: tensor<128x32xf32>) -> tensor<32x64xf32> {\n"
        "  %r = stablehlo.custom_call @fused_matmul_bias_activation(%a, %w) : (tensor<64x128xf32>, tensor<128x32xf32>) -> tensor<32x64xf32>\n"
        "  return %r : tensor<32x64xf32> }",
    "attention_result_not_q":
        "func.func @main(%q: tensor<2x64x32xf32>, %k: tensor<2x64x32xf32>, %v: tensor<2x64x32xf32>) -> tensor<2x32x32xf32> {\n"
        "  %r = stablehlo.custom_call @fused_scaled_dot_product_attention(%q, %k, %v) : (tensor<2x64x32xf32>, tensor<2x64x32xf32>, tensor<2x64x32xf32>) -> tensor<2x32x32xf32>\n"
        "  return %r : tensor<2x32x32xf32> }",
    "attention_q_other_type":
        "func.func @main(%q: tensor<2x64x32xbf16>, %k: tensor<2x64x32xf32>, %v: tensor<2x64x32xf32>) -> tensor<2x64x32xf32> {\n"
        "  %r = stablehlo.custom_call @fused_scaled_dot_product_attention(%q, %k, %v) : (tensor<2x64x32xbf16>, tensor<2x64x32xf32>, tensor<2x64x32xf32>) -> tensor<2x64x32xf32>\n"
        "  return %r : tensor<2x64x32xf32> }",
    "layer_norm_short_gamma":
        "func.func @main(%x: tensor<8x64xf32>, %g: tensor<32xf32>, %b: tensor<64xf32>) -> tensor<8x64xf32> {\n"
        "  %r = stablehlo.custom_call @fused_layer_norm(%x, %g, %b) : (tensor<8x64xf32>, tensor<32xf32>, tensor<64xf32>) -> tensor<8x64xf32>\n"
        "  return %r : tensor<8x64xf32> }",
}


@pytest.mark.parametrize("name", sorted(BAD_RESULT_TYPES))
@pytest.mark.parametrize("level", [0, 2])
def test_declared_result_types_are_checked_at_compile_time(sess, name, level):
    """A result (or operand) type the kernel would not honour is refused with PARSE_FAILED before
    anything can run: the kernels size their writes from the operands, not from the declaration.
    Host-only: these modules are never executed."""
    with pytest.raises(capi.MHLOError) as e:
        ops(sess, BAD_RESULT_TYPES[name], level)
    assert e.value.code == 3, (e.value.code, str(e.value))      # MHLO_ERROR_PARSE_FAILED


def test_erf_gelu_becomes_the_exact_fused_form(sess):
    """Both common spellings of 0.5 x (1 + erf(x / sqrt 2)) become a fused_gelu marked "erf": true
    (the executor then runs the exact function, not the tanh approximation); a wrong constant
    leaves the program as written; behind matmul + bias it is the "gelu_exact" epilogue."""
    assert ops(sess, M.GELU_ERF) == ["fused_gelu"] and ops(sess, M.GELU_ERF_MUL) == ["fused_gelu"]
    assert "erf" in ops(sess, M.GELU_ERF, 0)
    assert "fused_gelu" not in ops(sess, M.GELU_ERF.replace("1.41421354", "1.5"))
    assert "fused_gelu" not in ops(sess, M.GELU_ERF_MUL.replace("0.707106769", "0.7978845608"))
    assert "fused_gelu" not in ops(sess, M.GELU_ERF.replace("dense<2.0>", "dense<3.0>"))
    t = "tensor<32x128xf32>"
    text = (f"func.func @main(%x: tensor<32x64xf32>, %w: tensor<64x128xf32>, %b: tensor<128xf32>) -> {t} {{\n"
            f"  %d = stablehlo.dot_general %x, %w, contracting_dims = [1] x [0] : (tensor<32x64xf32>, tensor<64x128xf32>) -> {t}\n"
            f"  %bb = stablehlo.broadcast_in_dim %b, dims = [1] : (tensor<128xf32>) -> {t}\n"
            f"  %h = stablehlo.add %d, %bb : {t}\n"
            f"  %k = stablehlo.constant dense<0.707106769> : {t}\n  %one = stablehlo.constant dense<1.0> : {t}\n"
            f"  %half = stablehlo.constant dense<0.5> : {t}\n  %u = stablehlo.multiply %h, %k : {t}\n"
            f"  %e = chlo.erf %u : {t} -> {t}\n  %p = stablehlo.add %one, %e : {t}\n"
            f"  %hx = stablehlo.multiply %half, %h : {t}\n  %r = stablehlo.multiply %hx, %p : {t}\n  return %r : {t} }}")
    assert ops(sess, text) == ["fused_matmul_bias_activation"]


def test_one_pass_variance_layer_norm(sess):
    assert ops(sess, M.LAYER_NORM_ONE_PASS) == ["fused_layer_norm"]
    # the square of another mean, or a centring by another statistic, is not a LayerNorm
    assert "fused_layer_norm" not in ops(sess, M.LAYER_NORM_ONE_PASS.replace("%mm = stablehlo.multiply %mean, %mean", "%mm = stablehlo.multiply %mean, %m2"))
    assert "fused_layer_norm" not in ops(sess, M.LAYER_NORM_ONE_PASS.replace("broadcast_in_dim %mean, dims = [0]", "broadcast_in_dim %m2, dims = [0]"))


def test_silu_epilogue_and_unshifted_softmax(sess):
    t = "tensor<32x128xf32>"
    text = (f"func.func @main(%x: tensor<32x64xf32>, %w: tensor<64x128xf32>, %b: tensor<128xf32>) -> {t} {{\n"
            f"  %d = stablehlo.dot_general %x, %w, contracting_dims = [1] x [0] : (tensor<32x64xf32>, tensor<64x128xf32>) -> {t}\n"
            f"  %bb = stablehlo.broadcast_in_dim %b, dims = [1] : (tensor<128xf32>) -> {t}\n"
            f"  %h = stablehlo.add %d, %bb : {t}\n  %s = stablehlo.logistic %h : {t}\n"
            f"  %r = stablehlo.multiply %h, %s : {t}\n  return %r : {t} }}")
    assert ops(sess, text) == ["fused_matmul_bias_activation"]
    # the sigmoid is also a result: it must still be produced
    both = text.replace(f") -> {t} {{", f") -> ({t}, {t}) {{").replace(f"return %r : {t}", f"return %r, %s : {t}, {t}")
    assert "logistic" in ops(sess, both)
    unshifted = ("func.func @main(%x: tensor<8x32xf32>) -> tensor<8x32xf32> {\n"
                 "  %e = stablehlo.exponential %x : tensor<8x32xf32>\n  %zero = stablehlo.constant dense<0.0> : tensor<f32>\n"
                 "  %s = stablehlo.reduce(%e init: %zero) applies stablehlo.add across dimensions = [1] : (tensor<8x32xf32>, tensor<f32>) -> tensor<8xf32>\n"
                 "  %sb = stablehlo.broadcast_in_dim %s, dims = [0] : (tensor<8xf32>) -> tensor<8x32xf32>\n"
                 "  %r = stablehlo.divide %e, %sb : tensor<8x32xf32>\n  return %r : tensor<8x32xf32> }")
    assert ops(sess, unshifted) == ["fused_softmax"]


def test_calls_are_inlined(sess):
    """Private helper functions, a two-result call used as %r#0 / %r#1, calls inside callees, the
    entry function in the middle of the module: one flat program after parsing; a pattern that
    lives in a callee is recognised after inlining."""
    got = ops(sess, M.CALLS, 0)
    assert "call" not in got and sorted(got) == sorted(["add", "constant", "compare", "select", "negate", "multiply",
                                                        "constant", "compare", "select"])
    assert ops(sess, M.SOFTMAX_IN_CALLEE) == ["fused_softmax"]
    for bad, msg in ((M.CALLS.replace("call @relu_and_neg(%s)", "call @nowhere(%s)"), "unknown function"),
                     (M.CALLS.replace("%r = call @_where(%p, %a, %b)", "%r = call @_where_wrapper(%a, %b)")
                             .replace("(tensor<8x16xi1>, tensor<8x16xf32>, tensor<8x16xf32>) -> tensor<8x16xf32>\n    return %r : tensor<8x16xf32>\n  }\n}",
                                      "(tensor<8x16xf32>, tensor<8x16xf32>) -> tensor<8x16xf32>\n    return %r : tensor<8x16xf32>\n  }\n}"), "recursive"),
                     (M.CALLS.replace("%r:2 = call", "%r:3 = call"), "names 3 results"),
                     (M.CALLS.replace("call @relu_and_neg(%s) : (tensor<8x16xf32>)", "call @relu_and_neg(%s, %s) : (tensor<8x16xf32>, tensor<8x16xf32>)"), "takes 1 arguments")):
        with pytest.raises(capi.MHLOError) as e:
            ops(sess, bad, 0)
        assert e.value.code == 3 and msg in str(e.value), str(e.value)


def test_fused_ffn_custom_call(sess):
    assert ops(sess, M.FFN_CUSTOM_CALL.replace("ACT", "gelu")) == ["fused_ffn"]
    assert ops(sess, M.FFN_CUSTOM_CALL.replace("ACT", "gelu_exact")) == ["fused_ffn"]
    # as in the reference's handler, an activation it does not know means none and "is_gated" is ignored
    assert ops(sess, M.FFN_CUSTOM_CALL.replace("ACT", "mish")) == ["fused_ffn"]
    assert ops(sess, M.FFN_CUSTOM_CALL.replace('\\"ACT\\"', '\\"gelu\\", \\"is_gated\\": true')) == ["fused_ffn"]
    assert "is_gated" in M.FFN_CUSTOM_CALL.replace('\\"ACT\\"', '\\"gelu\\", \\"is_gated\\": true')
    with pytest.raises(capi.MHLOError):         # the down projection does not follow the up projection
        ops(sess, M.FFN_CUSTOM_CALL.replace("ACT", "gelu").replace("256x64xf32", "128x64xf32"))


def test_environment_switches_of_the_front_end(sess, tmp_path, capfd):
    """METALHLO_DISABLED_PASSES takes the reference's pass names (Compiler/PassManager.swift:154-201),
    METALHLO_DEBUG_PASSES=1 prints one line per pass, METALHLO_DUMP_OPTIMIZED=<file> receives the
    operation list after recognition."""
    block = M.transformer_block(2, 64, 4, 64, 256, "bf16")
    full = ops(sess, block)
    os.environ["METALHLO_DISABLED_PASSES"] = "residual-chain-fusion, transpose-folding"
    try:
        got = ops(sess, block)
        assert got.count("add") == 2 and "transpose" in got and got.count("fused_matmul_bias_activation") == 4
    finally:
        del os.environ["METALHLO_DISABLED_PASSES"]
    os.environ["METALHLO_DISABLED_PASSES"] = "softmax-fusion"
    try:
        got = ops(sess, block)        # no fused softmax, hence no fused attention either
        assert "fused_scaled_dot_product_attention" not in got and "exponential" in got and "fused_layer_norm" in got
    finally:
        del os.environ["METALHLO_DISABLED_PASSES"]
    assert ops(sess, block) == full
    dump = tmp_path / "opt.txt"
    os.environ["METALHLO_DUMP_OPTIMIZED"] = str(dump)
    os.environ["METALHLO_DEBUG_PASSES"] = "1"
    try:
        capfd.readouterr()
        ops(sess, M.SOFTMAX)
        err = capfd.readouterr().err
    finally:
        del os.environ["METALHLO_DUMP_OPTIMIZED"], os.environ["METALHLO_DEBUG_PASSES"]
    assert "[*] softmax-fusion ops: 9 -> 1" in err and "[ ] norm-fusion ops: 1 -> 1" in err
    text = dump.read_text()
    assert text.startswith("// optimized IR -- 1 ops") and "fused_softmax inputs=[%0]" in text and '"axis": 1' in text


def test_token_and_position_embedding_is_one_call(sess):
    """gather of whole table rows + a slice of the position table spread over the batch + the
    rounding: one kernel; the positions' first row travels in the configuration.  Left alone when
    the ids are i64, the gathered rows are a result too, or the slice cuts rows of the table."""
    assert ops(sess, M.embedding()) == ["fused_token_embedding"]
    assert ops(sess, M.embedding(dtype="f32", first=3)) == ["fused_token_embedding"]
    assert len(ops(sess, M.embedding(), 0)) == 5
    assert "fused_token_embedding" not in ops(sess, M.embedding(ids_type="i64"))
    assert "fused_token_embedding" not in ops(sess, M.embedding(keep_tokens=True))
    got = ops(sess, M.embedding(cols=80))
    assert got == ["slice", "fused_token_embedding"]          # the cut rows are made first, then used whole
    from metalhlo_amd import programs
    head = ops(sess, programs.gpt2_program(2, 64, 1, 4, 64, 1024, 1000, 128, "bf16"))
    assert head.count("fused_token_embedding") == 1 and "gather" not in head
    os.environ["METALHLO_DISABLED_PASSES"] = "embedding-fusion"
    try:
        assert ops(sess, M.embedding()) == ["gather", "slice", "broadcast_in_dim", "add", "convert"]
    finally:
        del os.environ["METALHLO_DISABLED_PASSES"]


def test_rope_and_elementwise_custom_calls_compile_and_reject(sess):
    """fused_rope and fused_elementwise (Compiler/CustomCallHandlers.swift:720-846, 927-1079): accepted forms and
    the handlers' own error cases, all decided at compile time."""
    assert ops(sess, M.rope_call()) == ["fused_rope"]
    assert ops(sess, M.rope_call(freq_cols=16)) == ["fused_rope"]
    assert ops(sess, M.rope_call(shape=(16, 32), dtype="bf16")) == ["fused_rope"]
    with pytest.raises(capi.MHLOError):          # an odd last axis cannot be split into halves
        ops(sess, M.rope_call(shape=(2, 16, 33), freq_cols=33))
    with pytest.raises(capi.MHLOError):          # frequencies of another width (the separate cos / sin form) are not served
        ops(sess, M.rope_call(freq_cols=8))
    with pytest.raises(capi.MHLOError) as e:     # one operand: CustomCallError.invalidInputCount(expected: 2, ...)
        ops(sess, M.rope_call().replace("(%x, %f)", "(%x)").replace("(tensor<2x3x16x32xf32>, tensor<16x32xf32>)", "(tensor<2x3x16x32xf32>)"))
    assert "expected 2" in str(e.value)
    assert ops(sess, M.elementwise_call(["add", "multiply"], 3)) == ["fused_elementwise"]
    assert ops(sess, M.elementwise_call(["tanh", "add", "negate"], 2, key="operations")) == ["fused_elementwise"]
    assert ops(sess, M.elementwise_call(["multiply", "exponential"], 2, dtype="bf16", scalar_inputs=(1,))) == ["fused_elementwise"]
    with pytest.raises(capi.MHLOError) as e:
        ops(sess, M.elementwise_call(["add", "atan2"], 3))
    assert "Unsupported operation in fused chain: atan2" in str(e.value)
    with pytest.raises(capi.MHLOError) as e:
        ops(sess, M.elementwise_call(["add", "multiply"], 2))
    assert "Not enough inputs" in str(e.value)
    with pytest.raises(capi.MHLOError) as e:
        ops(sess, M.elementwise_call(["add"], 2).replace("ops", "steps"))
    assert "Missing 'ops' or 'operations'" in str(e.value)
    # sine, cosine, floor and ceil are also plain operations of the front end now
    text = """func.func @main(%x: tensor<8xf32>) -> tensor<8xf32> {
      %0 = stablehlo.sine %x : tensor<8xf32>
      %1 = stablehlo.cosine %0 : tensor<8xf32>
      %2 = stablehlo.floor %1 : tensor<8xf32>
      %3 = stablehlo.ceil %2 : tensor<8xf32>
      return %3 : tensor<8xf32> }"""
    assert ops(sess, text) == ["sine", "cosine", "floor", "ceil"]


def test_batch_norm_and_depth_attention_custom_calls_compile_and_reject(sess):
    """fused_batch_norm and fused_depth_attention (Compiler/CustomCallHandlers.swift:414-452, 1084-1140): accepted
    forms and the handlers' own operand-count errors, decided at compile time."""
    assert ops(sess, M.batch_norm_call()) == ["fused_batch_norm"]
    assert ops(sess, M.batch_norm_call(shape=(64, 30), dtype="bf16", eps=0.001)) == ["fused_batch_norm"]
    with pytest.raises(capi.MHLOError) as e:     # CustomCallError.invalidInputCount(expected: 5, ...)
        ops(sess, M.batch_norm_call(n_operands=4))
    assert "expected 5" in str(e.value)
    with pytest.raises(capi.MHLOError):          # a statistics vector of another length
        ops(sess, M.batch_norm_call().replace("%m: tensor<16xf32>", "%m: tensor<8xf32>").replace(
            "tensor<16xf32>, tensor<16xf32>) ->", "tensor<8xf32>, tensor<16xf32>) ->"))
    assert ops(sess, M.depth_attention_call()) == ["fused_depth_attention"]
    assert ops(sess, M.depth_attention_call(lead=(2, 3), depth=32, hidden=768, dtype="bf16", scale=0.036)) == ["fused_depth_attention"]
    assert ops(sess, M.depth_attention_call(query_row=False)) == ["fused_depth_attention"]
    with pytest.raises(capi.MHLOError) as e:     # more stored rows than the kernel holds scores for
        ops(sess, M.depth_attention_call(depth=65))
    assert "64" in str(e.value)
    with pytest.raises(capi.MHLOError) as e:
        ops(sess, M.depth_attention_call().replace("(%q, %k, %v)", "(%q, %k)").replace(
            "(tensor<4x1x32xf32>, tensor<4x8x32xf32>, tensor<4x8x32xf32>)", "(tensor<4x1x32xf32>, tensor<4x8x32xf32>)"))
    assert "expected 3" in str(e.value)
