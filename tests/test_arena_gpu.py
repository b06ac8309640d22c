"""GPU: executions out of the arena and replays of the captured HIP graph give the results
of the per-value allocation path bit for bit, for every replay, with other work on the
device between the replays; the counters of mhlo_ext_executable_plan show which path ran."""
import ctypes as C

import numpy as np
import pytest

from tests import fusion_modules as fm
from tests.test_arena_host import chain

pytestmark = pytest.mark.gpu

FAN = """func.func @main(%x: tensor<128x128xf32>, %y: tensor<128x128xf32>) -> (tensor<128x128xf32>, tensor<128x128xf32>) {
  %a = stablehlo.tanh %x : tensor<128x128xf32>
  %b = stablehlo.exponential %y : tensor<128x128xf32>
  %c = stablehlo.negate %x : tensor<128x128xf32>
  %d = stablehlo.abs %y : tensor<128x128xf32>
  %ab = stablehlo.add %a, %b : tensor<128x128xf32>
  %cd = stablehlo.multiply %c, %d : tensor<128x128xf32>
  %t = stablehlo.transpose %cd, dims = [1, 0] : (tensor<128x128xf32>) -> tensor<128x128xf32>
  %m = stablehlo.dot_general %ab, %t, contracting_dims = [1] x [0] : (tensor<128x128xf32>, tensor<128x128xf32>) -> tensor<128x128xf32>
  %r = stablehlo.add %m, %ab : tensor<128x128xf32>
  return %r, %ab : tensor<128x128xf32>, tensor<128x128xf32>
}"""

PASS_THROUGH = """func.func @main(%x: tensor<8x8xf32>) -> (tensor<8x8xf32>, tensor<8x8xf32>, tensor<64xf32>) {
  %a = stablehlo.tanh %x : tensor<8x8xf32>
  %r = stablehlo.reshape %a : (tensor<8x8xf32>) -> tensor<64xf32>
  return %x, %a, %r : tensor<8x8xf32>, tensor<8x8xf32>, tensor<64xf32>
}"""


@pytest.fixture(scope="module")
def sess():
    from metalhlo_amd import capi
    s = capi.Session()
    yield s
    s.close()


def run_with(sess, exe, bufs):
    n_out = sess.lib.mhlo_executable_output_count(exe)
    outs = (C.c_void_p * max(n_out, 1))()
    got = C.c_int32()
    arr = (C.c_void_p * max(len(bufs), 1))(*bufs)
    rc = sess.lib.mhlo_execute(exe, arr, len(bufs), outs, C.byref(got))
    assert rc == 0, sess.lib.mhlo_get_last_error()
    res = [sess.to_numpy(outs[i]) for i in range(got.value)]
    for i in range(got.value):
        sess.lib.mhlo_buffer_destroy(outs[i])
    return res


def inputs_for(rng, text):
    import re
    sig = text[text.index("@main(") + 6:text.index(") ->")]
    out = []
    for shape, et in re.findall(r"tensor<((?:\d+x)*)(\w+)>", sig):
        dims = [int(d) for d in shape.split("x") if d]
        a = rng.standard_normal(dims).astype(np.float32)
        if et == "bf16":
            a = (a.view(np.uint32) >> 16).astype(np.uint16)
        out.append((a, et))
    return out


MODULES = {"chain": (chain(9), 2), "fan": (FAN, 2), "layer_norm_unfused": (fm.LAYER_NORM, 0), "layer_norm": (fm.LAYER_NORM, 2),
           "softmax_unfused": (fm.SOFTMAX, 0), "ffn_up": (fm.FFN_UP, 2), "pass_through": (PASS_THROUGH, 2)}


@pytest.mark.parametrize("name", sorted(MODULES))
def test_arena_and_graph_match_per_value_allocation(name, sess, monkeypatch):
    text, opt = MODULES[name]
    rng = np.random.default_rng(5)
    ins = inputs_for(rng, text)
    monkeypatch.setenv("METALHLO_ARENA", "0")
    exe = sess.compile(text, opt_level=opt)
    want = sess.run(exe, ins)
    assert sess.plan(exe)["eager_runs"] == 1
    sess.lib.mhlo_executable_destroy(exe)

    monkeypatch.setenv("METALHLO_ARENA", "1")
    monkeypatch.setenv("METALHLO_HIP_GRAPH", "0")
    exe = sess.compile(text, opt_level=opt)
    for _ in range(3):
        got = sess.run(exe, ins)
        assert all(np.array_equal(g, w, equal_nan=True) for g, w in zip(got, want))
    p = sess.plan(exe)
    assert p["planned"] == 1 and p["eager_runs"] == 3 and p["graph_captures"] == 0
    sess.lib.mhlo_executable_destroy(exe)

    monkeypatch.setenv("METALHLO_HIP_GRAPH", "1")
    exe = sess.compile(text, opt_level=opt)
    other = sess.compile(chain(3), opt_level=2)
    bufs = [sess.buffer(a, t) for a, t in ins]
    for i in range(6):
        got = run_with(sess, exe, bufs)
        assert all(np.array_equal(g, w, equal_nan=True) for g, w in zip(got, want)), f"replay {i}"
        sess.run(other, [(rng.standard_normal((64, 64)).astype(np.float32), "f32")])     # eager work and a sync between replays
    p = sess.plan(exe)
    assert p["eager_runs"] == 1 and p["graph_captures"] == 1 and p["graph_replays"] == 5, p
    # new contents at new addresses: captured again (or replayed when the pool hands the old addresses
    # back), and still right
    ins2 = inputs_for(np.random.default_rng(6), text)
    monkeypatch.setenv("METALHLO_ARENA", "0")
    ref = sess.compile(text, opt_level=opt)
    want2 = sess.run(ref, ins2)
    sess.lib.mhlo_executable_destroy(ref)
    monkeypatch.setenv("METALHLO_ARENA", "1")
    bufs2 = [sess.buffer(a, t) for a, t in ins2]
    for i in range(3):
        got = run_with(sess, exe, bufs2)
        assert all(np.array_equal(g, w, equal_nan=True) for g, w in zip(got, want2)), f"second set, replay {i}"
        got = run_with(sess, exe, bufs)
        assert all(np.array_equal(g, w, equal_nan=True) for g, w in zip(got, want)), f"first set again, replay {i}"
    p = sess.plan(exe)
    assert p["graph_captures"] == 2 and p["graph_replays"] == 11 and p["eager_runs"] == 1, p
    for b in bufs + bufs2:
        sess.lib.mhlo_buffer_destroy(b)
    sess.lib.mhlo_executable_destroy(exe)
    sess.lib.mhlo_executable_destroy(other)


def test_graph_is_the_default_at_optimisation_level_three(sess, monkeypatch):
    monkeypatch.delenv("METALHLO_HIP_GRAPH", raising=False)
    monkeypatch.delenv("METALHLO_ARENA", raising=False)
    x = np.random.default_rng(1).standard_normal((64, 64)).astype(np.float32)
    for opt, n_ops, captures in ((2, 20, 0), (3, 20, 1), (3, 5, 0)):     # short programs stay eager
        exe = sess.compile(chain(n_ops), opt_level=opt)
        buf = sess.buffer(x, "f32")
        outs = [run_with(sess, exe, [buf])[0] for _ in range(3)]
        assert np.array_equal(outs[0], outs[1]) and np.array_equal(outs[0], outs[2])
        assert sess.plan(exe)["graph_captures"] == captures
        sess.lib.mhlo_buffer_destroy(buf)
        sess.lib.mhlo_executable_destroy(exe)


def test_attention_program_replays(sess, monkeypatch):
    """The fused attention + RMSNorm program in bf16 through the graph path, against the eager one."""
    text = """func.func @main(%q: tensor<2x4x256x64xbf16>, %k: tensor<2x4x256x64xbf16>, %v: tensor<2x4x256x64xbf16>, %g: tensor<64xbf16>) -> tensor<2x4x256x64xbf16> {
        %0 = stablehlo.custom_call @fused_scaled_dot_product_attention(%q, %k, %v) {backend_config = "{\\"scale\\": 0.125, \\"is_causal\\": true}"} : (tensor<2x4x256x64xbf16>, tensor<2x4x256x64xbf16>, tensor<2x4x256x64xbf16>) -> tensor<2x4x256x64xbf16>
        %1 = stablehlo.custom_call @fused_rms_norm(%0, %g) {backend_config = "{\\"eps\\": 1e-6, \\"axes\\": [-1]}"} : (tensor<2x4x256x64xbf16>, tensor<64xbf16>) -> tensor<2x4x256x64xbf16>
        return %1 : tensor<2x4x256x64xbf16> }"""
    ins = inputs_for(np.random.default_rng(9), text)
    monkeypatch.setenv("METALHLO_ARENA", "0")
    exe = sess.compile(text)
    want = sess.run(exe, ins)[0]
    sess.lib.mhlo_executable_destroy(exe)
    monkeypatch.setenv("METALHLO_ARENA", "1")
    monkeypatch.setenv("METALHLO_HIP_GRAPH", "1")
    exe = sess.compile(text)
    bufs = [sess.buffer(a, t) for a, t in ins]
    for i in range(4):
        assert np.array_equal(run_with(sess, exe, bufs)[0], want), f"replay {i}"
    assert sess.plan(exe)["graph_replays"] == 3
    for b in bufs:
        sess.lib.mhlo_buffer_destroy(b)
    sess.lib.mhlo_executable_destroy(exe)


def test_replay_results_are_handed_out_without_a_copy_and_never_overwritten(sess, monkeypatch):
    """A captured graph writes its results into buffers of their own.  While the caller still holds
    the results of a replay the next execution must not run that graph (it would overwrite them):
    it gets a second and then a third graph with result buffers of their own (a loop that keeps
    the previous step's output alive replays every step), with all three sets held it runs
    eagerly, the held buffers keep their contents, and once they are released the graphs are
    replayed again.  Programs that return an input or an alias keep the copy-out form (covered
    by 'pass_through' above)."""
    monkeypatch.setenv("METALHLO_ARENA", "1")
    monkeypatch.setenv("METALHLO_HIP_GRAPH", "1")
    rng = np.random.default_rng(21)
    ins = inputs_for(rng, FAN)
    exe = sess.compile(FAN)
    bufs = [sess.buffer(a, t) for a, t in ins]
    other = [sess.buffer(a + 1.0, t) for a, t in ins]           # a second set of inputs -> a second graph
    want = run_with(sess, exe, bufs)                             # the first execution is eager
    want_other = run_with(sess, exe, other)                      # captured and replayed at once
    for i in range(3):                                           # capture, then replays: results released each time
        got = run_with(sess, exe, bufs)
        assert all(np.array_equal(g, w) for g, w in zip(got, want)), f"replay {i}"
    base = sess.plan(exe)
    assert base["graph_captures"] == 2 and base["graph_replays"] == 4 and base["eager_runs"] == 1

    def execute_keep(inputs):
        outs = (C.c_void_p * 2)()
        n = C.c_int32()
        arr = (C.c_void_p * len(inputs))(*inputs)
        assert sess.lib.mhlo_execute(exe, arr, len(inputs), outs, C.byref(n)) == 0, sess.lib.mhlo_get_last_error()
        return [outs[i] for i in range(n.value)]

    held = [execute_keep(bufs)]                                  # a replay whose results stay with the caller
    assert sess.plan(exe)["graph_replays"] == 5
    held.append(execute_keep(bufs))                              # must not touch held[0]: a second result set
    held.append(execute_keep(bufs))                              # ... and a third
    p3 = sess.plan(exe)
    assert p3["graph_replays"] == 7 and p3["eager_runs"] == 1 and p3["graph_captures"] == 4, p3
    held.append(execute_keep(bufs))                              # all three sets held: eager
    after = sess.plan(exe)
    assert after["graph_replays"] == 7 and after["eager_runs"] == 2 and after["graph_captures"] == 4, after
    got_other = run_with(sess, exe, other)                       # other inputs: their own graph, their own result buffers
    assert all(np.array_equal(g, w) for g, w in zip(got_other, want_other))
    for hs in held:
        vals = [sess.to_numpy(h) for h in hs]
        assert all(np.array_equal(g, w) for g, w in zip(vals, want))
    # the pattern of a loop that holds step n while it runs step n + 1: every step is a replay
    for h in held[1] + held[2] + held[3]:
        sess.lib.mhlo_buffer_destroy(h)
    prev = held[0]
    for i in range(6):
        cur = execute_keep(bufs)
        assert all(np.array_equal(sess.to_numpy(h), w) for h, w in zip(cur, want)), f"rotating replay {i}"
        assert all(np.array_equal(sess.to_numpy(h), w) for h, w in zip(prev, want)), f"held result during rotating replay {i}"
        for h in prev:
            sess.lib.mhlo_buffer_destroy(h)
        prev = cur
    for h in prev:
        sess.lib.mhlo_buffer_destroy(h)
    end = sess.plan(exe)
    assert end["graph_replays"] == 14 and end["eager_runs"] == 2 and end["graph_captures"] == 4, end
    for b in bufs + other:
        sess.lib.mhlo_buffer_destroy(b)
    sess.lib.mhlo_executable_destroy(exe)
