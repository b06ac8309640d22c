"""The reference's own benchmark programs (tests/golden/benchmark_modules.json, extracted from its
benchmark suite by tests/golden/make_benchmark_modules.py) through the C API: what the pattern
recogniser makes of them (CPU) and, on the GPU, the fused and the as-written runs against a
float64 restatement of each program built from the oracle's operators."""
import json
import os
from collections import Counter

import numpy as np
import pytest

os.environ.setdefault("METALHLO_ALLOW_NO_DEVICE", "1")
from metalhlo_amd import capi   # noqa: E402
from oracle import oracle       # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))
MODULES = {e["id"]: e for e in json.load(open(os.path.join(HERE, "golden", "benchmark_modules.json")))}

# operations left after recognition (reshapes are views and launch nothing)
EXPECTED = {
    "ATTN-002": {"fused_scaled_dot_product_attention": 1},
    "NORM-LN-002": {"fused_layer_norm": 1},
    "NORM-LN-004": {"fused_layer_norm": 1},
    "XFMR-INF-001": {"reshape": 8, "dot_general": 4, "fused_scaled_dot_product_attention": 1},
    "XFMR-INF-004": {"reshape": 2, "fused_matmul_bias_activation": 2},
    "XFMR-INF-005": {"fused_softmax": 1},
    "XFMR-INF-006": {"fused_layer_norm": 2, "reshape": 8, "dot_general": 4, "fused_scaled_dot_product_attention": 1, "add": 2,
                     "fused_matmul_bias_activation": 2},
}


@pytest.fixture(scope="module")
def sess():
    s = capi.Session()
    yield s
    s.close()


@pytest.mark.parametrize("bench_id", sorted(MODULES))
def test_recogniser_on_the_reference_benchmark_programs(sess, bench_id):
    exe = sess.compile(MODULES[bench_id]["mlir"])
    got = Counter(sess.ops(exe))
    sess.lib.mhlo_executable_destroy(exe)
    assert dict(got) == EXPECTED[bench_id]
    exe = sess.compile(MODULES[bench_id]["mlir"], 0)           # level 0 keeps the program as written
    assert not any(o.startswith("fused_") for o in sess.ops(exe))
    sess.lib.mhlo_executable_destroy(exe)


def _inputs(entry, seed):
    """The distributions the reference's generators use, except that tensors it fills with zeros
    (biases, beta) get small values, so that a dropped bias shows."""
    rng = np.random.default_rng(seed)
    out = []
    for spec in entry["inputs"]:
        shape = spec["shape"]
        if spec["dist"] == "uniform":
            a = rng.uniform(spec["lo"], spec["hi"], shape)
        elif spec["dist"] == "normal":
            a = rng.normal(spec["mean"], spec["std"], shape)
        else:
            a = rng.normal(0.0, 0.05, shape)
        out.append(a.astype(np.float32))
    return out


def _ln(x, g, b):
    return oracle.layer_norm(x, g, b, 1e-5)


def _silu(v):
    return v / (1.0 + np.exp(-v))


def _attention_block(x2, wq, wk, wv, wo, heads=12, hd=64):
    """Projections, the reference programs' head "split" (a plain reshape of [S, H*D] to [1,H,S,D]),
    softmax(q k^T / 8) v, the reshape back and the output projection."""
    S = x2.shape[0]
    q, k, v = (oracle.gemm(x2, w).reshape(1, heads, S, hd) for w in (wq, wk, wv))
    a = oracle.attention(q, k, v, scale=0.125)
    return oracle.gemm(a.reshape(S, heads * hd), wo)


def _expected(bench_id, a):
    a = [t.astype(np.float64) for t in a]
    if bench_id == "ATTN-002":
        return oracle.attention(a[0], a[1], a[2], scale=0.125)
    if bench_id.startswith("NORM-LN"):
        return _ln(*a)
    if bench_id == "XFMR-INF-005":
        return oracle.softmax(a[0])
    if bench_id == "XFMR-INF-004":
        x, w1, b1, w2, b2 = a
        h = _silu(oracle.gemm(x.reshape(-1, 768), w1) + b1)
        return (oracle.gemm(h, w2) + b2).reshape(x.shape)
    if bench_id == "XFMR-INF-001":
        x, wq, wk, wv, wo = a
        return _attention_block(x[0], wq, wk, wv, wo).reshape(x.shape)
    if bench_id == "XFMR-INF-006":
        x, g1, b1, wq, wk, wv, wo, g2, b2, w1, c1, w2, c2 = a
        res1 = x + _attention_block(_ln(x, g1, b1)[0], wq, wk, wv, wo).reshape(x.shape)
        h = _silu(oracle.gemm(_ln(res1, g2, b2)[0], w1) + c1)
        return res1 + (oracle.gemm(h, w2) + c2).reshape(x.shape)
    raise KeyError(bench_id)


@pytest.mark.gpu
@pytest.mark.parametrize("bench_id", sorted(MODULES))
def test_reference_benchmark_programs_match_the_oracle(bench_id):
    """fp32 programs: a single fused operator is held to 1e-5, the chained programs (projections,
    attention, LayerNorms, feed-forward: up to ten fp32 operators in a row) to 5e-5, the bound the
    transformer-block test uses.  Prints the time of one execution for the record."""
    s = capi.Session()
    try:
        entry = MODULES[bench_id]
        arrays = _inputs(entry, seed=42)
        exp = _expected(bench_id, arrays)
        tol = 1e-5 if EXPECTED[bench_id].keys() <= {"fused_layer_norm", "fused_softmax", "fused_scaled_dot_product_attention"} else 5e-5
        for level in (None, 0):
            exe = s.compile(entry["mlir"], level)
            (got,) = s.run(exe, [(a, "f32") for a in arrays])
            err = np.abs(got.astype(np.float64) - exp)
            lim = np.maximum(tol, tol * np.abs(exp))
            assert (err <= lim).all(), f"{bench_id} level {level}: worst error / limit {np.max(err / lim):.2f}"
            if level is None:
                # the reference's benchmarks report GPU time with the inputs resident (gpuTime of its
                # timing struct): the same here, median of ten executions after two warm-up ones
                import ctypes as C
                bufs = [s.buffer(a, "f32") for a in arrays]
                arr = (C.c_void_p * len(bufs))(*bufs)
                outs, n_out = (C.c_void_p * 1)(), C.c_int32()
                enc, gpu, tot = C.c_double(), C.c_double(), C.c_double()
                times = []
                for i in range(12):
                    assert s.lib.mhlo_execute_with_timing(exe, arr, len(bufs), outs, C.byref(n_out), C.byref(enc), C.byref(gpu),
                                                          C.byref(tot)) == 0
                    s.lib.mhlo_buffer_destroy(outs[0])
                    if i >= 2:
                        times.append(gpu.value)
                for b in bufs:
                    s.lib.mhlo_buffer_destroy(b)
                print(f"[benchmark module] {bench_id} ({entry['name']}): {sorted(times)[len(times) // 2] * 1e3:.3f} ms GPU time per "
                      f"execution, inputs resident; the reference publishes {entry['published']}", flush=True)
            s.lib.mhlo_executable_destroy(exe)
    finally:
        s.close()
