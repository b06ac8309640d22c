"""GPU parity: GPT-2-small forward through the fused pipeline (bf16 compute,
fp32 parameters) vs the float64 oracle with the same rounding points.
Tolerance: bf16 rule, |got - e| <= max(2e-2, 2e-2 |e|)."""
import numpy as np
import pytest
import torch

from oracle import oracle
from tests.util import as_f64

pytestmark = pytest.mark.gpu


def _check(got, exp, what="", frac=1e-5):
    """Every fused operator is held to 2e-2 on its own (other test files).  Through a
    whole network a value that sits next to a bf16 rounding boundary can round the
    other way than in the float64 oracle and the difference is carried on, so the
    end-to-end rule is: at most `frac` of the logits outside the 2e-2 rule (1e-5 for
    the 2-layer model, 5e-3 for 12 layers, where the residual stream reaches
    magnitudes whose bf16 spacing is itself 3e-2), an RMS error below 1e-2, and none
    outside 5e-2, the bound the reference's own bf16 suite uses
    (Examples/FlaxExample/flax_metalhlo_bf16.py:68).  The measured figures are printed
    (pytest -s / -rP shows them) so that the distance to each limit can be read off a run."""
    g = as_f64(got)
    err = np.abs(g - exp)
    frac_bad = float((err > np.maximum(2e-2, 2e-2 * np.abs(exp))).mean())
    worst = float((err / np.maximum(1.0, np.abs(exp))).max())
    rms = float(np.sqrt((err ** 2).mean()))
    print(f"[gpt2 parity] {what}: {g.size} logits, fraction outside 2e-2 = {frac_bad:.3e} (limit {frac:.0e}), "
          f"worst scaled error = {worst:.4f} (limit 0.05), rms = {rms:.5f} (limit 0.01), "
          f"rms of the logits = {float(np.sqrt((exp ** 2).mean())):.4f}", flush=True)
    assert frac_bad <= frac and worst <= 5e-2 and rms <= 1e-2, \
        f"{what}: {frac_bad:.2e} of logits outside 2e-2, worst scaled error {worst:.4f}, rms {rms:.4f}"


def test_gpt2_reduced_depth_full_width():
    """2 layers, full width / heads / vocabulary, B2 S192: whole-tensor comparison."""
    from metalhlo_amd.gpt2 import GPT2, GPT2Config, init_params
    cfg = GPT2Config(n_layer=2)
    params = init_params(cfg, seed=5)
    rng = np.random.default_rng(5)
    ids = rng.integers(0, cfg.vocab, (2, 192)).astype(np.int32)
    model = GPT2(cfg, params)
    logits = model.forward(torch.from_numpy(ids).cuda())
    assert logits.shape == (2, 192, cfg.vocab) and logits.dtype == torch.bfloat16
    exp = oracle.gpt2_forward(ids, params, cfg.n_head, "bf16")
    _check(logits, exp, what="2-layer GPT-2")


def test_gpt2_small_baseline_shape():
    """The benchmark configuration: 12 layers, B8 S1024.  The oracle runs on two of the eight
    sequences (they are independent); properties cover the rest."""
    from metalhlo_amd.gpt2 import GPT2, GPT2Config, init_params
    cfg = GPT2Config()
    params = init_params(cfg, seed=5)
    rng = np.random.default_rng(5)
    ids = rng.integers(0, cfg.vocab, (8, 1024)).astype(np.int32)
    model = GPT2(cfg, params)
    dev_ids = torch.from_numpy(ids).cuda()
    logits = model.forward(dev_ids)
    assert logits.shape == (8, 1024, cfg.vocab)
    assert torch.isfinite(logits.float()).all()
    # two batch elements against the oracle: every position of the first 256 of sequence 0 and,
    # through the full causal prefix of sequence 5, its first 64 and last 64 positions
    exp = oracle.gpt2_forward(ids[:1, :256], params, cfg.n_head, "bf16")      # causal: prefix suffices
    _check(logits[:1, :256], exp, what="GPT-2-small, sequence 0, positions 0-255", frac=5e-3)
    exp5 = oracle.gpt2_forward(ids[5:6], params, cfg.n_head, "bf16")
    pos = np.r_[0:64, 960:1024]
    _check(logits[5:6][:, pos], exp5[:, pos], what="GPT-2-small, sequence 5, positions 0-63 and 960-1023", frac=5e-3)
    del exp5
    # causality: changing the last token of every sequence leaves earlier logits bit-identical
    ids2 = ids.copy(); ids2[:, -1] = (ids2[:, -1] + 1) % cfg.vocab
    l2 = model.forward(torch.from_numpy(ids2).cuda())
    assert torch.equal(l2[:, :-1], logits[:, :-1]) and not torch.equal(l2[:, -1], logits[:, -1])
    # batch independence: sequence 3 alone gives the same logits as inside the batch
    l3 = model.forward(dev_ids[3:4].contiguous())
    assert torch.equal(l3[0], logits[3])
    # greedy next-token ids are exact integer results of argmax over bf16 logits
    from metalhlo_amd import kernels
    nxt = kernels.argmax(logits[:, -1].contiguous())
    assert torch.equal(nxt.long(), logits[:, -1].float().argmax(-1))


def test_gpt2_small_fp32_compute_full_depth():
    """The same 12-layer model computed in fp32 (fp32 GEMM and attention on the fp32 matrix
    instruction, fp32 row kernels): one full sequence of 1024 positions against the float64
    oracle with fp32 rounding points.  No bf16 rounding decides anything here, so this pins the
    structure of the pipeline at full size (layer order, residuals, head split, causal
    attention over the whole sequence, tied head) at a bar two hundred times tighter than the
    bf16 rule.  Limit 1e-4 scaled (|got - e| <= 1e-4 max(1, |e|)); measured: worst 6.0e-6, rms
    9.7e-7 (printed by the test)."""
    from metalhlo_amd.gpt2 import GPT2, GPT2Config, init_params
    cfg = GPT2Config()
    params = init_params(cfg, seed=5)
    ids = np.random.default_rng(5).integers(0, cfg.vocab, (8, 1024)).astype(np.int32)[2:3]
    model = GPT2(cfg, params, compute_dtype=torch.float32)
    logits = model.forward(torch.from_numpy(np.ascontiguousarray(ids)).cuda())
    assert logits.shape == (1, 1024, cfg.vocab) and logits.dtype == torch.float32
    exp = oracle.gpt2_forward(ids, params, cfg.n_head, "f32")
    err = np.abs(as_f64(logits) - exp) / np.maximum(1.0, np.abs(exp))
    print(f"[gpt2 parity] fp32 compute, 12 layers, sequence 2, 1024 positions: worst scaled error {err.max():.3e} "
          f"(limit 1e-4), rms {np.sqrt((err ** 2).mean()):.3e}", flush=True)
    assert err.max() <= 1e-4


def test_gpt2_graph_replay_matches_eager():
    """A captured forward pass replayed several times, with eager work and
    synchronisations between the replays, reproduces the eager logits bit for bit."""
    from metalhlo_amd.gpt2 import GPT2, GPT2Config, init_params
    cfg = GPT2Config(n_layer=2, d_model=128, n_head=4, d_ff=512, vocab=1000, n_pos=64)
    model = GPT2(cfg, init_params(cfg, seed=11))
    rng = np.random.default_rng(12)
    ids = [torch.from_numpy(rng.integers(0, cfg.vocab, (2, 64)).astype(np.int32)).cuda() for _ in range(4)]
    graphed = model.capture(ids[0])
    for k in (0, 1, 2, 3, 1):
        eager = model.forward(ids[k]).clone()
        torch.cuda.synchronize()
        got = graphed(ids[k]).clone()
        torch.cuda.synchronize()
        assert torch.equal(got, eager), f"replay for ids[{k}] differs from the eager pass"
    with pytest.raises(ValueError):
        graphed(ids[0][:1])


def test_gpt2_small_from_text_through_the_c_api():
    """The benchmark program itself: the 12-layer GPT-2 forward at B8 S1024 as ONE plain StableHLO
    module (fp32 parameters, no custom calls), compiled by mhlo_compile at level 3 and run three
    times through mhlo_execute — the first execution issues the launches eagerly, the second
    captures them, the third replays the HIP graph.  Every execution's logits ([8,1024,50257],
    rows at odd byte offsets) are compared on sampled positions with the float64 oracle by the
    end-to-end rule, the three executions with each other bit for bit, and the replay with the
    hand-written pipeline of metalhlo_amd.gpt2 (>= 99.5 % of the sampled logits within 2e-2)."""
    import ctypes
    from metalhlo_amd import capi, programs
    from metalhlo_amd.gpt2 import GPT2, GPT2Config, init_params
    cfg = GPT2Config()
    B, S = 8, 1024
    params = init_params(cfg, seed=5)
    ids = np.random.default_rng(5).integers(0, cfg.vocab, (B, S)).astype(np.int32)
    text = programs.gpt2_program(B, S, cfg.n_layer, cfg.n_head, cfg.d_model // cfg.n_head, cfg.d_ff, cfg.vocab, cfg.n_pos)
    sess = capi.Session()
    exe = sess.compile(text, opt_level=3)
    ops = sess.ops(exe)
    assert ops.count("fused_scaled_dot_product_attention") == 12 and ops.count("fused_layer_norm") == 25
    arrs = [(ids, "i32"), (params["wte"], "f32"), (params["wpe"], "f32")]
    for l in params["layers"]:
        arrs += [(l[n], "f32") for n in programs.GPT2_LAYER_PARAMS]
    arrs += [(params["lnf_g"], "f32"), (params["lnf_b"], "f32")]
    bufs = [sess.buffer(a, t) for a, t in arrs]
    arr = (ctypes.c_void_p * len(bufs))(*bufs)
    outs = (ctypes.c_void_p * 1)()
    got = ctypes.c_int32()
    runs = []
    for _ in range(3):
        assert sess.lib.mhlo_execute(exe, arr, len(bufs), outs, ctypes.byref(got)) == 0, sess.lib.mhlo_get_last_error()
        assert got.value == 1
        bits = torch.from_numpy(sess.to_numpy(outs[0]).view(np.int16))     # bf16 bit patterns [8,1024,50257]
        sess.lib.mhlo_buffer_destroy(outs[0])
        runs.append(bits)
    plan = sess.plan(exe)
    assert plan.get("graph_replays", 0) >= 1 and plan.get("eager_runs", 0) >= 1, plan
    assert torch.equal(runs[0], runs[1]) and torch.equal(runs[1], runs[2]), "eager, captured and replayed executions differ"
    logits = runs[2].view(torch.bfloat16)
    assert logits.shape == (B, S, cfg.vocab)
    exp = oracle.gpt2_forward(ids[:1, :256], params, cfg.n_head, "bf16")
    _check(logits[:1, :256], exp, what="GPT-2-small from text, sequence 0, positions 0-255", frac=5e-3)
    exp5 = oracle.gpt2_forward(ids[5:6], params, cfg.n_head, "bf16")
    pos = np.r_[0:64, 960:1024]
    _check(logits[5:6][:, pos], exp5[:, pos], what="GPT-2-small from text, sequence 5, positions 0-63 and 960-1023", frac=5e-3)
    del exp, exp5
    for b in bufs:
        sess.lib.mhlo_buffer_destroy(b)
    sess.lib.mhlo_executable_destroy(exe)
    sess.close()
    hand = GPT2(cfg, params).forward(torch.from_numpy(ids).cuda())
    for sl in (np.s_[0, :256], np.s_[5, 960:], np.s_[7, 500:564]):
        a, h = as_f64(logits[sl]), as_f64(hand[sl])
        err = np.abs(a - h)
        assert (err <= np.maximum(2e-2, 2e-2 * np.abs(h))).mean() >= 0.995, sl
