"""GPU: StableHLO text in -> results out through the mhlo_* C API, checked against
the expectations the reference's own op-level tests hold and against the oracle.
fp32 tolerance 1e-5 (rule max(tol, tol*|e|)), bf16 2e-2."""
import ctypes as C
import json

import numpy as np
import pytest

from oracle import oracle

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


def bf16(a):
    return oracle.bf16_round_bits(np.asarray(a, np.float32))


def unbf16(bits):
    return oracle.bf16_bits_to_f32(bits).astype(np.float64)


def test_add_dot_and_dot_general(sess):
    # Tests/MetalHLOTests/OperationTests.swift:327-349 and TrainingOpsTests.swift:14-139
    exe = sess.compile("""module @dot { func.func @main(%arg0: tensor<2x3xf32>, %arg1: tensor<3x2xf32>) -> (tensor<2x2xf32>) {
        %0 = stablehlo.dot %arg0, %arg1 : (tensor<2x3xf32>, tensor<3x2xf32>) -> tensor<2x2xf32>
        return %0 : tensor<2x2xf32> } }""")
    a = np.array([[1, 2, 3], [4, 5, 6]], np.float32)
    b = np.array([[1, 2], [3, 4], [5, 6]], np.float32)
    (r,) = sess.run(exe, [(a, "f32"), (b, "f32")])
    assert np.array_equal(r, [[22, 28], [49, 64]])
    exe = sess.compile("""func.func @main(%lhs: tensor<2x3x4xf32>, %rhs: tensor<2x4x5xf32>) -> (tensor<2x3x5xf32>) {
        %0 = stablehlo.dot_general %lhs, %rhs, #stablehlo.dot<lhs_batching_dimensions = [0], rhs_batching_dimensions = [0], lhs_contracting_dimensions = [2], rhs_contracting_dimensions = [1]> : (tensor<2x3x4xf32>, tensor<2x4x5xf32>) -> tensor<2x3x5xf32>
        return %0 : tensor<2x3x5xf32> }""")
    rng = np.random.default_rng(61)
    l, r_ = rng.uniform(-1, 1, (2, 3, 4)).astype(np.float32), rng.uniform(-1, 1, (2, 4, 5)).astype(np.float32)
    (r,) = sess.run(exe, [(l, "f32"), (r_, "f32")])
    close(r, oracle.dot_general(l, r_, [0], [0], [2], [1]), 1e-5)
    exe = sess.compile("""func.func @main(%lhs: tensor<4x3xf32>, %rhs: tensor<5x4xf32>) -> (tensor<3x5xf32>) {
        %0 = stablehlo.dot_general %lhs, %rhs, #stablehlo.dot<lhs_batching_dimensions = [], rhs_batching_dimensions = [], lhs_contracting_dimensions = [0], rhs_contracting_dimensions = [1]> : (tensor<4x3xf32>, tensor<5x4xf32>) -> tensor<3x5xf32>
        return %0 : tensor<3x5xf32> }""")
    l = np.array([[1, 5, 9], [2, 6, 10], [3, 7, 11], [4, 8, 12]], np.float32)
    (r,) = sess.run(exe, [(l, "f32"), (np.ones((5, 4), np.float32), "f32")])
    assert np.array_equal(r, [[10] * 5, [26] * 5, [42] * 5])
    # contracting a middle dimension forces a transposing copy in front of the GEMM
    exe = sess.compile("""func.func @main(%l: tensor<3x4x2xf32>, %r: tensor<2x4x5xf32>) -> tensor<3x2x2x5xf32> {
        %0 = stablehlo.dot_general %l, %r, batching_dims = [] x [], contracting_dims = [1] x [1] : (tensor<3x4x2xf32>, tensor<2x4x5xf32>) -> tensor<3x2x2x5xf32>
        return %0 : tensor<3x2x2x5xf32> }""")
    l, r_ = rng.uniform(-1, 1, (3, 4, 2)).astype(np.float32), rng.uniform(-1, 1, (2, 4, 5)).astype(np.float32)
    (r,) = sess.run(exe, [(l, "f32"), (r_, "f32")])
    close(r, oracle.dot_general(l, r_, [], [], [1], [1]), 1e-5)


def test_decomposed_softmax_and_gelu(sess):
    # Tests/MetalHLOTests/ActivationOpsTests.swift:137-192 and :252-318 (module text restated)
    exe = sess.compile("""module @softmax { func.func @main(%x: tensor<4xf32>) -> (tensor<4xf32>) {
        %init_max = stablehlo.constant dense<-1e38> : tensor<f32>
        %max_val = stablehlo.reduce %x, %init_max applies stablehlo.maximum across dimensions = [0] : (tensor<4xf32>, tensor<f32>) -> tensor<f32>
        %mb = stablehlo.broadcast_in_dim %max_val, dims = [] : (tensor<f32>) -> tensor<4xf32>
        %sh = stablehlo.subtract %x, %mb : tensor<4xf32>
        %e = stablehlo.exponential %sh : tensor<4xf32>
        %zero = stablehlo.constant dense<0.0> : tensor<f32>
        %s = stablehlo.reduce %e, %zero applies stablehlo.add across dimensions = [0] : (tensor<4xf32>, tensor<f32>) -> tensor<f32>
        %sb = stablehlo.broadcast_in_dim %s, dims = [] : (tensor<f32>) -> tensor<4xf32>
        %r = stablehlo.divide %e, %sb : tensor<4xf32>
        return %r : tensor<4xf32> } }""")
    (r,) = sess.run(exe, [(np.array([1, 2, 3, 4], np.float32), "f32")])
    close(r, oracle.softmax(np.array([1.0, 2, 3, 4])), 1e-5)
    assert abs(r.sum() - 1) < 1e-5
    exe = sess.compile("""module @gelu { func.func @main(%x: tensor<6xf32>) -> (tensor<6xf32>) {
        %half = stablehlo.constant dense<0.5> : tensor<6xf32>
        %one = stablehlo.constant dense<1.0> : tensor<6xf32>
        %coeff = stablehlo.constant dense<0.044715> : tensor<6xf32>
        %k = stablehlo.constant dense<0.7978845608> : tensor<6xf32>
        %x2 = stablehlo.multiply %x, %x : tensor<6xf32>
        %x3 = stablehlo.multiply %x2, %x : tensor<6xf32>
        %cx3 = stablehlo.multiply %coeff, %x3 : tensor<6xf32>
        %inner = stablehlo.add %x, %cx3 : tensor<6xf32>
        %sc = stablehlo.multiply %k, %inner : tensor<6xf32>
        %t = stablehlo.tanh %sc : tensor<6xf32>
        %opt = stablehlo.add %one, %t : tensor<6xf32>
        %hx = stablehlo.multiply %half, %x : tensor<6xf32>
        %r = stablehlo.multiply %hx, %opt : tensor<6xf32>
        return %r : tensor<6xf32> } }""")
    x = np.array([-2, -1, 0, 1, 2, 3], np.float32)
    (r,) = sess.run(exe, [(x, "f32")])
    close(r, oracle.gelu_tanh(x.astype(np.float64)), 1e-4)
    assert abs(r[2]) < 1e-6 and r[5] > 2.9


def test_config0_fused_sdpa_module(sess):
    """The first benchmark configuration: single StableHLO module for fused SDPA, fp32 B1 H4 S128 D64,
    causal, scale 1/8, N(0,1) inputs (seed 1234): causal flag and additive-mask forms."""
    rng = np.random.default_rng(1234)
    q, k, v = (rng.standard_normal((1, 4, 128, 64)).astype(np.float32) for _ in range(3))
    exp = oracle.attention(q, k, v, scale=0.125, is_causal=True)
    t = "tensor<1x4x128x64xf32>"
    cfg = json.dumps({"scale": 0.125, "has_mask": False, "is_causal": True}).replace('"', '\\"')
    exe = sess.compile(f"""module @sdpa {{ func.func @main(%q: {t}, %k: {t}, %v: {t}) -> ({t}) {{
        %0 = stablehlo.custom_call @fused_scaled_dot_product_attention(%q, %k, %v) {{backend_config = "{cfg}"}} : ({t}, {t}, {t}) -> {t}
        return %0 : {t} }} }}""")
    (o,) = sess.run(exe, [(q, "f32"), (k, "f32"), (v, "f32")])
    assert o.shape == (1, 4, 128, 64)
    close(o, exp, 1e-5)
    # the mask built inside the module: iota / compare / select, then has_mask
    cfg = json.dumps({"scale": 0.125, "has_mask": True}).replace('"', '\\"')
    exe = sess.compile(f"""func.func @main(%q: {t}, %k: {t}, %v: {t}) -> {t} {{
        %qi = stablehlo.iota dim = 0 : tensor<128x128xi32>
        %ki = stablehlo.iota dim = 1 : tensor<128x128xi32>
        %fut = stablehlo.compare GT, %ki, %qi, SIGNED : (tensor<128x128xi32>, tensor<128x128xi32>) -> tensor<128x128xi1>
        %ninf = stablehlo.constant dense<0xFF800000> : tensor<128x128xf32>
        %zero = stablehlo.constant dense<0.0> : tensor<128x128xf32>
        %m = stablehlo.select %fut, %ninf, %zero : tensor<128x128xi1>, tensor<128x128xf32>
        %0 = stablehlo.custom_call @fused_scaled_dot_product_attention(%q, %k, %v, %m) {{backend_config = "{cfg}"}} : ({t}, {t}, {t}, tensor<128x128xf32>) -> {t}
        return %0 : {t} }}""")
    (o,) = sess.run(exe, [(q, "f32"), (k, "f32"), (v, "f32")])
    close(o, exp, 1e-5)


def test_fused_custom_calls_bf16(sess):
    rng = np.random.default_rng(62)
    x = rng.standard_normal((64, 256)).astype(np.float32)
    g, b = (1 + 0.1 * rng.standard_normal(256)).astype(np.float32), (0.1 * rng.standard_normal(256)).astype(np.float32)
    w = (0.1 * rng.uniform(-1, 1, (256, 512))).astype(np.float32)
    bias = (0.02 * rng.standard_normal(512)).astype(np.float32)
    exe = sess.compile("""func.func @main(%x: tensor<64x256xbf16>, %g: tensor<256xbf16>, %b: tensor<256xbf16>, %w: tensor<256x512xbf16>, %bias: tensor<512xbf16>) -> (tensor<64x512xbf16>, tensor<64x256xbf16>, tensor<64x256xbf16>, tensor<64x256xbf16>) {
        %ln = stablehlo.custom_call @fused_layer_norm(%x, %g, %b) {backend_config = "{\\"eps\\": 1e-5, \\"axes\\": [-1]}"} : (tensor<64x256xbf16>, tensor<256xbf16>, tensor<256xbf16>) -> tensor<64x256xbf16>
        %up = stablehlo.custom_call @fused_matmul_bias_activation(%ln, %w, %bias) {backend_config = "{\\"activation\\": \\"gelu\\"}"} : (tensor<64x256xbf16>, tensor<256x512xbf16>, tensor<512xbf16>) -> tensor<64x512xbf16>
        %rms = stablehlo.custom_call @fused_rms_norm(%x, %g) {backend_config = "{\\"eps\\": 1e-6}"} : (tensor<64x256xbf16>, tensor<256xbf16>) -> tensor<64x256xbf16>
        %sm = stablehlo.custom_call @fused_softmax(%x) {backend_config = "{\\"axis\\": -1}"} : (tensor<64x256xbf16>) -> tensor<64x256xbf16>
        %ge = stablehlo.custom_call @fused_gelu(%x) {backend_config = "{\\"approximate\\": true}"} : (tensor<64x256xbf16>) -> tensor<64x256xbf16>
        return %up, %rms, %sm, %ge : tensor<64x512xbf16>, tensor<64x256xbf16>, tensor<64x256xbf16>, tensor<64x256xbf16> }""")
    ins = [(bf16(x), "bf16"), (bf16(g), "bf16"), (bf16(b), "bf16"), (bf16(w), "bf16"), (bf16(bias), "bf16")]
    up, rms, sm, ge = sess.run(exe, ins)
    X, G, B_, W, BI = (unbf16(bf16(a)) for a in (x, g, b, w, bias))
    ln = oracle.round_to(oracle.layer_norm(X, G, B_, 1e-5), "bf16")
    close(unbf16(up), oracle.matmul_bias_act(ln, W, BI, "gelu"), 2e-2)
    close(unbf16(rms), oracle.rms_norm(X, G, 1e-6), 2e-2)
    close(unbf16(sm), oracle.softmax(X), 2e-2)
    close(unbf16(ge), oracle.gelu_tanh(X), 2e-2)


def test_glue_ops_exact(sess):
    exe = sess.compile("""func.func @main(%x: tensor<4x6xf32>, %b: tensor<3xf32>, %ids: tensor<5xi32>, %tab: tensor<7x4xf32>) -> (tensor<2x3xbf16>, tensor<6x4xf32>, tensor<5x4xf32>, tensor<4xi32>) {
        %s = stablehlo.slice %x [1:3, 0:6:2] : (tensor<4x6xf32>) -> tensor<2x3xf32>
        %bb = stablehlo.broadcast_in_dim %b, dims = [1] : (tensor<3xf32>) -> tensor<2x3xf32>
        %a = stablehlo.add %s, %bb : tensor<2x3xf32>
        %c = stablehlo.convert %a : (tensor<2x3xf32>) -> tensor<2x3xbf16>
        %t = stablehlo.transpose %x, dims = [1, 0] : (tensor<4x6xf32>) -> tensor<6x4xf32>
        %g = "stablehlo.gather"(%tab, %ids) {dimension_numbers = #stablehlo.gather<offset_dims = [1], collapsed_slice_dims = [0], start_index_map = [0], index_vector_dim = 1>, slice_sizes = array<i64: 1, 4>} : (tensor<7x4xf32>, tensor<5xi32>) -> tensor<5x4xf32>
        %i = stablehlo.iota dim = 0 : tensor<4xi32>
        %two = stablehlo.constant dense<2> : tensor<4xi32>
        %m = stablehlo.multiply %i, %two : tensor<4xi32>
        return %c, %t, %g, %m : tensor<2x3xbf16>, tensor<6x4xf32>, tensor<5x4xf32>, tensor<4xi32> }""")
    rng = np.random.default_rng(63)
    x = rng.standard_normal((4, 6)).astype(np.float32)
    b = rng.standard_normal(3).astype(np.float32)
    ids = np.array([6, 0, 3, 3, 9], np.int32)       # 9 clamps to the last row
    tab = rng.standard_normal((7, 4)).astype(np.float32)
    c, t, g, m = sess.run(exe, [(x, "f32"), (b, "f32"), (ids, "i32"), (tab, "f32")])
    assert np.array_equal(c, bf16(x[1:3, 0:6:2] + b[None, :]))
    assert np.array_equal(t, x.T)
    assert np.array_equal(g, tab[np.clip(ids, 0, 6)])
    assert np.array_equal(m, [0, 2, 4, 6])


def test_stats_timing_profile_and_errors(sess):
    from metalhlo_amd import capi
    lib = sess.lib
    exe = sess.compile("""func.func @main(%a: tensor<2x3xf32>, %b: tensor<2x3xf32>) -> tensor<2x3xf32> {
        %0 = stablehlo.add %a, %b : tensor<2x3xf32>
        return %0 : tensor<2x3xf32> }""")
    a = np.arange(6, dtype=np.float32).reshape(2, 3)
    for _ in range(3):
        (r,) = sess.run(exe, [(a, "f32"), (a, "f32")])
        assert np.array_equal(r, 2 * a)
    st = capi.ExecutionStats()
    assert lib.mhlo_executable_get_stats(exe, C.byref(st)) == 0
    assert st.execution_count == 3 and st.total_execution_time_ms > 0
    assert abs(st.average_execution_time_ms - st.total_execution_time_ms / 3) < 1e-9
    lib.mhlo_executable_reset_stats(exe)
    lib.mhlo_executable_get_stats(exe, C.byref(st))
    assert st.execution_count == 0
    ba, bb = sess.buffer(a, "f32"), sess.buffer(a, "f32")
    ins = (C.c_void_p * 2)(ba, bb)
    outs = (C.c_void_p * 1)()
    n = C.c_int32()
    enc, gpu, tot = C.c_double(), C.c_double(), C.c_double()
    assert lib.mhlo_execute_with_timing(exe, ins, 2, outs, C.byref(n), C.byref(enc), C.byref(gpu), C.byref(tot)) == 0
    assert n.value == 1 and 0 < enc.value <= gpu.value <= tot.value < 5.0          # seconds
    lib.mhlo_buffer_destroy(outs[0])
    prof = capi.ExecutionProfile()
    assert lib.mhlo_execute_with_profile(exe, ins, 2, outs, C.byref(n), C.byref(prof)) == 0
    assert (prof.partition_count, prof.gpu_partition_count, prof.ane_partition_count, prof.used_ane) == (1, 1, 0, False)
    # too-small destination and input mismatches
    small = np.empty(3, np.float32)
    assert lib.mhlo_buffer_to_host(outs[0], small.ctypes.data_as(C.c_void_p), small.nbytes) == 9
    assert lib.mhlo_buffer_byte_count(outs[0]) == 24 and lib.mhlo_buffer_element_type(outs[0]) == 1
    lib.mhlo_buffer_destroy(outs[0])
    assert lib.mhlo_execute(exe, ins, 1, outs, C.byref(n)) == 7
    wrong = sess.buffer(np.zeros((3, 2), np.float32), "f32")
    ins2 = (C.c_void_p * 2)(ba, wrong)
    assert lib.mhlo_execute(exe, ins2, 2, outs, C.byref(n)) == 7
    name = lib.mhlo_client_device_name(sess.client)
    assert b"gfx950" in C.string_at(name)
    lib.mhlo_free_string(name)
    for b in (ba, bb, wrong):
        lib.mhlo_buffer_destroy(b)
    lib.mhlo_executable_destroy(exe)


def test_per_operation_device_times(sess, monkeypatch):
    """mhlo_execute_with_profile times the execution it makes operation by operation (HIP events
    around every operation's launches); mhlo_ext_executable_profile returns the list: one entry per
    launched operation in program order with its result shape, all times positive and their sum
    no more than the execution's total.  The results are those of an ordinary execution, and the
    next ordinary execution is not profiled (at level 3 it may be replayed as a graph again)."""
    from metalhlo_amd import capi
    text = """func.func @main(%x: tensor<64x256xf32>, %w: tensor<256x128xf32>) -> tensor<64x128xf32> {
        %0 = stablehlo.custom_call @fused_softmax(%x) {backend_config = "{\\"axis\\": -1}"} : (tensor<64x256xf32>) -> tensor<64x256xf32>
        %1 = stablehlo.dot %0, %w : (tensor<64x256xf32>, tensor<256x128xf32>) -> tensor<64x128xf32>
        %2 = stablehlo.tanh %1 : tensor<64x128xf32>
        %3 = stablehlo.add %2, %1 : tensor<64x128xf32>
        return %3 : tensor<64x128xf32> }"""
    exe = sess.compile(text)
    rng = np.random.default_rng(77)
    x, w = rng.standard_normal((64, 256)).astype(np.float32), rng.standard_normal((256, 128)).astype(np.float32) * 0.1
    (want,) = sess.run(exe, [(x, "f32"), (w, "f32")])
    assert sess.profile(exe) == []
    bufs = [sess.buffer(x, "f32"), sess.buffer(w, "f32")]
    arr = (C.c_void_p * 2)(*bufs)
    outs = (C.c_void_p * 1)()
    n = C.c_int32()
    prof = capi.ExecutionProfile()
    assert sess.lib.mhlo_execute_with_profile(exe, arr, 2, outs, C.byref(n), C.byref(prof)) == 0
    got = sess.to_numpy(outs[0])
    sess.lib.mhlo_buffer_destroy(outs[0])
    assert np.array_equal(got, want)
    times = sess.profile(exe)
    assert [t[0] for t in times] == ["fused_softmax", "dot", "tanh", "add"]
    assert [t[1] for t in times] == ["64x256xf32", "64x128xf32", "64x128xf32", "64x128xf32"]
    assert all(t[2] > 0 for t in times) and sum(t[2] for t in times) * 1e-3 <= prof.total_time_ms
    assert prof.partition_count == 1 and prof.gpu_time_ms > 0
    # METALHLO_PROFILE_GPU=1 profiles ordinary executions too
    monkeypatch.setenv("METALHLO_PROFILE_GPU", "1")
    assert sess.lib.mhlo_execute(exe, arr, 2, outs, C.byref(n)) == 0
    sess.lib.mhlo_buffer_destroy(outs[0])
    assert len(sess.profile(exe)) == 4
    for b in bufs:
        sess.lib.mhlo_buffer_destroy(b)
    sess.lib.mhlo_executable_destroy(exe)
