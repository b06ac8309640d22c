"""GPU: one whole pre-LayerNorm transformer block written in plain StableHLO (93 operations, no
custom calls; tests/fusion_modules.py transformer_block) through mhlo_compile: the pattern
recogniser turns it into LayerNorm / GEMM+bias(+GELU) / attention kernels plus the head
split and merge glue (18 operations; the causal mask built from iotas becomes the causal flag, the residual adds go into GEMM epilogues), and both that and the program run as written agree with
the float64 oracle of the block.  f32: |got - e| <= max(tol, tol |e|) with tol 5e-5 for the
whole block (about ten chained operators, each held to 1e-5 on its own); bf16: the
end-to-end rule used for the GPT-2 logits (99.5 % within 2e-2, worst 6e-2)."""
import ctypes as C

import numpy as np
import pytest
import torch  # noqa: F401  (before the C API library: torch brings its own HIP runtime, and the first one loaded serves the process)

from oracle import oracle
from tests import fusion_modules as fm
from tests.test_arena_gpu import run_with

pytestmark = pytest.mark.gpu

B, S, H, D, F = 2, 64, 4, 32, 256
d = H * D
FUSED = ["fused_layer_norm", "fused_matmul_bias_activation", "slice", "reshape", "transpose", "slice", "reshape", "transpose",
         "slice", "reshape", "transpose", "fused_scaled_dot_product_attention", "transpose", "reshape", "fused_matmul_bias_activation",
         "fused_layer_norm", "fused_matmul_bias_activation", "fused_matmul_bias_activation"]


@pytest.fixture(scope="module")
def sess():
    from metalhlo_amd import capi
    s = capi.Session()
    yield s
    s.close()


def block_inputs(seed):
    rng = np.random.default_rng(seed)
    n = lambda *shape, s=1.0: (s * rng.standard_normal(shape)).astype(np.float32)
    return [n(B, S, d), 1 + n(d, s=0.1), n(d, s=0.1), n(d, 3 * d, s=d ** -0.5), n(3 * d, s=0.1), n(d, d, s=d ** -0.5), n(d, s=0.1),
            1 + n(d, s=0.1), n(d, s=0.1), n(d, F, s=d ** -0.5), n(F, s=0.1), n(F, d, s=F ** -0.5), n(d, s=0.1)]


def block_oracle_d(ins, Dh):
    x, g1, b1, wqkv, bqkv, wo, bo, g2, b2, w1, c1, w2, c2 = (np.asarray(a, dtype=np.float64) for a in ins)
    dd = H * Dh
    h = oracle.layer_norm(x, g1, b1, 1e-5)
    qkv = oracle.matmul_bias_act(h.reshape(B * S, dd), wqkv, bqkv).reshape(B, S, 3, H, Dh)
    q, k, v = (qkv[:, :, i].transpose(0, 2, 1, 3) for i in range(3))
    o = oracle.attention(q, k, v, scale=Dh ** -0.5, is_causal=True)
    o = o.transpose(0, 2, 1, 3).reshape(B * S, dd)
    r1 = x + oracle.matmul_bias_act(o, wo, bo).reshape(B, S, dd)
    h2 = oracle.layer_norm(r1, g2, b2, 1e-5)
    up = oracle.matmul_bias_act(h2.reshape(B * S, dd), w1, c1, "gelu")
    return r1 + oracle.matmul_bias_act(up, w2, c2).reshape(B, S, dd)


def block_oracle(*ins):
    return block_oracle_d(ins, D)


def test_block_f32_fused_and_as_written(sess, monkeypatch):
    text = fm.transformer_block(B, S, H, D, F, "f32")
    ins = block_inputs(11)
    exp = block_oracle(*ins)
    fused, plain = sess.compile(text), sess.compile(text, 0)
    assert sess.ops(fused) == FUSED
    assert len(sess.ops(plain)) == 93 and not any(o.startswith("fused_") for o in sess.ops(plain))
    args = [(a, "f32") for a in ins]
    for exe in (fused, plain):
        (got,) = sess.run(exe, args)
        err = np.abs(got.astype(np.float64) - exp)
        assert np.all(err <= np.maximum(5e-5, 5e-5 * np.abs(exp))), err.max()
    # the program as written is long enough for graph replay: replays equal the eager run bit for bit
    monkeypatch.setenv("METALHLO_HIP_GRAPH", "1")
    graphed = sess.compile(text, 0)
    bufs = [sess.buffer(a, t) for a, t in args]
    (want,) = sess.run(plain, args)
    for i in range(4):
        assert np.array_equal(run_with(sess, graphed, bufs)[0], want), f"replay {i}"
    p = sess.plan(graphed)
    assert p["graph_captures"] == 1 and p["graph_replays"] == 3 and p["arena_bytes"] < p["unshared_bytes"] // 4
    for b in bufs:
        sess.lib.mhlo_buffer_destroy(b)
    for exe in (fused, plain, graphed):
        sess.lib.mhlo_executable_destroy(exe)


def test_block_bf16_fused(sess):
    text = fm.transformer_block(B, S, H, D, F, "bf16")
    ins = [oracle.bf16_bits_to_f32(oracle.bf16_round_bits(a)) for a in block_inputs(12)]     # what the kernels see
    exp = block_oracle(*ins)
    exe = sess.compile(text)
    assert sess.ops(exe) == FUSED
    (got,) = sess.run(exe, [(oracle.bf16_round_bits(a), "bf16") for a in ins])
    sess.lib.mhlo_executable_destroy(exe)
    err = np.abs(oracle.bf16_bits_to_f32(got).astype(np.float64) - exp)
    ok = err <= np.maximum(2e-2, 2e-2 * np.abs(exp))
    assert ok.mean() >= 0.995 and np.all(err <= np.maximum(6e-2, 6e-2 * np.abs(exp))), (ok.mean(), err.max())


def test_block_bf16_attention_reads_the_projection_in_place(sess):
    """With a 16-bit type and D = 64 the head split (slice / reshape / transpose of the fused QKV
    projection) and the head merge are not run at all: attention reads its operands as strided
    views of the projection and writes [B,S,H,D] directly.  Seven operations remain, one kernel each, and the
    result equals the one with the glue materialised (same kernels, same order of arithmetic)."""
    Dh = 64
    text = fm.transformer_block(B, S, H, Dh, F, "bf16")
    rng = np.random.default_rng(13)
    dd = H * Dh
    n = lambda *shape, s=1.0: oracle.bf16_round_bits((s * rng.standard_normal(shape)).astype(np.float32))
    ins = [n(B, S, dd), n(dd, s=0.1), n(dd, s=0.1), n(dd, 3 * dd, s=dd ** -0.5), n(3 * dd, s=0.1), n(dd, dd, s=dd ** -0.5), n(dd, s=0.1),
           n(dd, s=0.1), n(dd, s=0.1), n(dd, F, s=dd ** -0.5), n(F, s=0.1), n(F, dd, s=F ** -0.5), n(dd, s=0.1)]
    ins[1] = oracle.bf16_round_bits(1 + oracle.bf16_bits_to_f32(ins[1]))
    ins[7] = oracle.bf16_round_bits(1 + oracle.bf16_bits_to_f32(ins[7]))
    args = [(a, "bf16") for a in ins]
    fused, plain = sess.compile(text), sess.compile(text, 0)
    assert sess.ops(fused) == ["fused_layer_norm", "fused_matmul_bias_activation", "fused_scaled_dot_product_attention",
                               "fused_matmul_bias_activation", "fused_layer_norm", "fused_matmul_bias_activation",
                               "fused_matmul_bias_activation"]
    (a,), (b,) = sess.run(fused, args), sess.run(plain, args)
    sess.lib.mhlo_executable_destroy(fused)
    sess.lib.mhlo_executable_destroy(plain)
    fa, fb = oracle.bf16_bits_to_f32(a).astype(np.float64), oracle.bf16_bits_to_f32(b).astype(np.float64)
    # against the program run operation by operation (bf16 after every one of its 93 operations)
    err = np.abs(fa - fb)
    ok = err <= np.maximum(2e-2, 2e-2 * np.abs(fb))
    assert ok.mean() >= 0.995 and np.all(err <= np.maximum(6e-2, 6e-2 * np.abs(fb))), (ok.mean(), err.max())
    # against the float64 oracle of the block
    f = [oracle.bf16_bits_to_f32(x) for x in ins]
    exp = block_oracle_d(f, Dh)
    err = np.abs(fa - exp)
    ok = err <= np.maximum(2e-2, 2e-2 * np.abs(exp))
    assert ok.mean() >= 0.995 and np.all(err <= np.maximum(6e-2, 6e-2 * np.abs(exp))), (ok.mean(), err.max())


def test_gpt2_program_through_the_c_api(sess):
    """A whole GPT-2 forward (reduced: 2 layers, d 256, vocab 1000) as one plain StableHLO module with
    fp32 parameters: compiled by mhlo_compile it runs as gather + per layer twelve parameter
    converts and the seven fused kernels, and its logits follow the float64 oracle of the model
    (the end-to-end rule of the bf16 GPT-2 tests) and the hand-written forward of metalhlo_amd.gpt2."""
    from metalhlo_amd.gpt2 import GPT2, GPT2Config, init_params
    cfg = GPT2Config(vocab=1000, n_pos=128, d_model=256, n_head=4, n_layer=2, d_ff=1024)
    Bq, Sq = 2, 64
    params = init_params(cfg, seed=21)
    rng = np.random.default_rng(22)
    for lyr in params["layers"]:                      # non-trivial biases and LayerNorm parameters
        for name, a in lyr.items():
            if a.ndim == 1:
                lyr[name] = (a + 0.05 * rng.standard_normal(a.shape)).astype(np.float32)
    ids = rng.integers(0, cfg.vocab, (Bq, Sq)).astype(np.int32)
    text = fm.gpt2_program(Bq, Sq, cfg.n_layer, cfg.n_head, cfg.d_model // cfg.n_head, cfg.d_ff, cfg.vocab, cfg.n_pos)
    exe = sess.compile(text)
    ops = sess.ops(exe)
    assert ops.count("fused_scaled_dot_product_attention") == 2 and ops.count("fused_matmul_bias_activation") == 8
    assert ops.count("fused_layer_norm") == 5 and not {"reduce", "exponential", "tanh", "transpose", "select"} & set(ops)
    args = [(ids, "i32"), (params["wte"], "f32"), (params["wpe"], "f32")]
    for lyr in params["layers"]:
        args += [(lyr[n], "f32") for n in fm.GPT2_LAYER_PARAMS]
    args += [(params["lnf_g"], "f32"), (params["lnf_b"], "f32")]
    (got,) = sess.run(exe, args)
    sess.lib.mhlo_executable_destroy(exe)
    got = oracle.bf16_bits_to_f32(got).astype(np.float64)
    exp = oracle.gpt2_forward(ids, params, cfg.n_head, "bf16")
    err = np.abs(got - exp)
    ok = err <= np.maximum(2e-2, 2e-2 * np.abs(exp))
    assert got.shape == (Bq, Sq, cfg.vocab) and ok.mean() >= 0.995 and np.all(err <= np.maximum(6e-2, 6e-2 * np.abs(exp))), (ok.mean(), err.max())
    hand = GPT2(cfg, params).forward(torch.from_numpy(ids).cuda()).float().cpu().numpy().astype(np.float64)
    err = np.abs(got - hand)
    assert (err <= np.maximum(2e-2, 2e-2 * np.abs(hand))).mean() >= 0.995
