#!/usr/bin/env python3
"""Benchmark of the fused-kernel hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--only]

One "step" is one launch of the workload's kernel over one batch of synthetic
input that already sits in HBM.  The headline workload is the bf16 GEMM 4096^3
(fp32 accumulate, the second benchmark configuration); the other kernels of the path
(flash attention, softmax, LayerNorm, RMSNorm, bias+GELU) are timed the same way
and reported under "kernels" of the same JSON line unless --only is given.

Timing: HIP events recorded on the stream the kernels are launched on, around
exactly K launches, after W warm-up launches, bracketed by device
synchronisation.  `roofline.achieved` = algorithmic FLOPs (or bytes) per launch
divided by the mean launch duration from those events.  A device that has idled
needs tens of milliseconds of work before it holds its clocks, far more than five
warm-up launches of a 100 us kernel; `--ramp-ms` (default 150, reported as
`clock_ramp_ms`, 0 switches it off) keeps the device busy with the same kernel for
that long before the W warm-up launches of every workload.
`cpu_baseline` (per kernel) times the same operator on the host cores with torch's
CPU kernels, and for the GEMM also the C restatement under oracle/, each on a
bounded sample of the workload (never part of the measured GPU path).
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0       # MI355X HBM3E
PEAK_CLOCK_MHZ = 2400.0     # the shader clock the matrix peak is quoted at

# HBM bytes per launch from rocprofv3 FETCH_SIZE + WRITE_SIZE, each scaled by what the same
# counter reads for the 'copy' workload (256 MiB in, 256 MiB out); see profiles/<workload>.txt.
# TRAFFIC_COMMIT: the commit of this repository the counter runs were taken at (the profiles say so too).
TRAFFIC_COMMIT = "78f698b"
MEASURED_TRAFFIC = {
    "gemm": 237458425,
    "gemm_f32": 812880561,
    "attention": 753138116,
    "attention_full": 268936609,
    "attention_f32": 1879189489,
    "softmax": 536739646,
    "layer_norm": 536883062,
    "rms_norm": 536780726,
    "bias_gelu": 536741693,
    "copy": 536870912,
}


RAMP_MS = 0.0


def _ramp(fn, torch):
    """Keeps the device busy with fn for RAMP_MS milliseconds (untimed)."""
    if RAMP_MS <= 0:
        return
    t0 = time.perf_counter()
    i = 0
    while (time.perf_counter() - t0) * 1e3 < RAMP_MS:
        for _ in range(8):
            fn(i)
            i += 1
        torch.cuda.synchronize()


def _time_launches(fn, steps, warmup, torch):
    """Times exactly `steps` launches of fn(i) after `warmup` untimed ones, with HIP events on the
    current stream: one event in front of the first launch and one behind every launch.  Returns
    (mean seconds per launch from the first event to the last, host wall seconds per launch,
    sorted per-launch seconds from consecutive events, (t0, t1) host clock around the timed region)."""
    for i in range(warmup):
        fn(i)
    torch.cuda.synchronize()
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
    t0 = time.perf_counter()
    ev[0].record()
    for i in range(steps):
        fn(i)
        ev[i + 1].record()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    each = sorted(ev[i].elapsed_time(ev[i + 1]) * 1e-3 for i in range(steps))
    return ev[0].elapsed_time(ev[steps]) * 1e-3 / steps, (t1 - t0) / steps, each, (t0, t1)


class DeviceSampler:
    """Board power and shader clock from the amdgpu hwmon files of the first card that has them,
    read by a side thread every millisecond or so while a workload runs.  The controller averages
    power over milliseconds, so the figures describe the steady state of the loop the sampler runs
    beside (ramp, warm-up and timed launches of one kernel), not a single launch."""

    def __init__(self):
        import glob
        self.power = self.cap = self.freq = self.dpm = None
        for d in sorted(glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*")):
            for name in ("power1_average", "power1_input"):
                if self.power is None and os.path.exists(os.path.join(d, name)):
                    self.power = os.path.join(d, name)
            if self.power and self.power.startswith(d):
                if os.path.exists(os.path.join(d, "power1_cap")):
                    self.cap = os.path.join(d, "power1_cap")
                if os.path.exists(os.path.join(d, "freq1_input")):
                    self.freq = os.path.join(d, "freq1_input")
                else:       # the level table of the shader clock; the current level carries a star
                    dpm = os.path.join(os.path.dirname(os.path.dirname(d)), "pp_dpm_sclk")
                    self.dpm = dpm if os.path.exists(dpm) else None
                break
        self.samples = []
        self._stop = None

    @staticmethod
    def _read(path):
        try:
            with open(path) as f:
                return float(f.read().strip())
        except (OSError, ValueError):
            return None

    def _clock_hz(self):
        if self.freq:
            return self._read(self.freq)
        if self.dpm:
            try:
                with open(self.dpm) as f:
                    for line in f:
                        if "*" in line:
                            return float(line.split(":")[1].strip().split("Mhz")[0]) * 1e6
            except (OSError, ValueError, IndexError):
                return None
        return None

    def available(self):
        return self.power is not None and self._read(self.power) is not None

    def start(self):
        import threading
        self.samples = []
        self._stop = threading.Event()

        def loop():
            while not self._stop.is_set():
                w = self._read(self.power)
                f = self._clock_hz()
                self.samples.append((time.perf_counter(), w, f))
                time.sleep(0.001)
        self._th = threading.Thread(target=loop, daemon=True)
        self._th.start()

    def stop(self, since=None):
        """Mean power (W) and clock (MHz) of the samples taken after host time `since`."""
        self._stop.set()
        self._th.join()
        sel = [s for s in self.samples if since is None or s[0] >= since] or self.samples[-3:]
        ws = [s[1] for s in sel if s[1] is not None]
        fs = [s[2] for s in sel if s[2] is not None]
        cap = self._read(self.cap) if self.cap else None
        return dict(power_w=round(sum(ws) / len(ws) / 1e6, 1) if ws else None,
                    power_cap_w=round(cap / 1e6, 1) if cap else None,
                    clock_mhz=round(sum(fs) / len(fs) / 1e6) if fs else None, samples=len(sel))


# ---------------------------------------------------------------- workloads
def _rng_dev(torch, draw, dtype):
    """A host array drawn from numpy's generator (the seeds and distributions of the benchmark
    configurations) -> device tensor of `dtype`, rounded to nearest even."""
    return torch.from_numpy(draw).to("cuda").to(dtype)


def wl_gemm(torch, kernels, M=4096, N=4096, K=4096):
    import numpy as np
    rng = np.random.default_rng(2)
    a = _rng_dev(torch, rng.uniform(-1, 1, (M, K)).astype(np.float32), torch.bfloat16)
    b = _rng_dev(torch, rng.uniform(-1, 1, (K, N)).astype(np.float32), torch.bfloat16)
    c = torch.empty(M, N, dtype=torch.bfloat16, device="cuda")
    return dict(name=f"bf16 GEMM {M}x{N}x{K} (row-major A[M,K], B[K,N]; fp32 accumulate, bf16 out)",
                fn=lambda i: kernels.matmul(a, b, out=c), flops=2.0 * M * N * K,
                bytes=2.0 * (M * K + K * N + M * N), bound="mfma", kernel="gemm256_kernel")


PEAK_F32_TFLOPS = 157.3    # MI355X dense fp32 MFMA


def wl_gemm_f32(torch, kernels, M=4096, N=4096, K=4096):
    import numpy as np
    rng = np.random.default_rng(2)
    a = _rng_dev(torch, rng.uniform(-1, 1, (M, K)).astype(np.float32), torch.float32)
    b = _rng_dev(torch, rng.uniform(-1, 1, (K, N)).astype(np.float32), torch.float32)
    c = torch.empty(M, N, dtype=torch.float32, device="cuda")
    return dict(name=f"fp32 GEMM {M}x{N}x{K} (row-major A[M,K], B[K,N]; fp32 operands and accumulate on the fp32 matrix instruction)",
                fn=lambda i: kernels.matmul(a, b, out=c), flops=2.0 * M * N * K, bytes=4.0 * (M * K + K * N + M * N),
                bound="mfma", peak=PEAK_F32_TFLOPS, kernel="gemm_f32_mfma_kernel")


def wl_attention(torch, kernels, B=4, H=32, S=4096, D=128, causal=True, fp32=False):
    import numpy as np
    rng = np.random.default_rng(4)
    dt = torch.float32 if fp32 else torch.bfloat16
    q, k, v = (_rng_dev(torch, rng.standard_normal((B, H, S, D), dtype=np.float32), dt) for _ in range(3))
    flops = 4.0 * B * H * S * S * D * (0.5 if causal else 1.0)
    r = dict(name=f"{'fp32' if fp32 else 'bf16'} flash-attention fwd B{B} H{H} S{S} D{D} {'causal' if causal else 'full'}",
             fn=lambda i: kernels.flash_attention(q, k, v, is_causal=causal), flops=flops,
             bytes=4.0 * B * H * S * D * (4 if fp32 else 2), bound="mfma", kernel="fa_f32_mfma_kernel" if fp32 else "fa_pipe_kernel")
    if fp32:
        r["peak"] = PEAK_F32_TFLOPS
    return r


def _rows(torch, rows=32768, cols=4096, nbuf=3):
    # several input sets, visited round-robin, so that a launch cannot find its
    # input still resident in the 256 MB last-level cache from the previous one
    import numpy as np
    rng = np.random.default_rng(3)
    bf = torch.bfloat16
    xs = [_rng_dev(torch, rng.standard_normal((rows, cols), dtype=np.float32), bf) for _ in range(nbuf)]
    gam = _rng_dev(torch, (1 + 0.1 * rng.standard_normal(cols)).astype(np.float32), bf)
    bet = _rng_dev(torch, (0.1 * rng.standard_normal(cols)).astype(np.float32), bf)
    bias = _rng_dev(torch, (0.02 * rng.standard_normal(cols)).astype(np.float32), bf)
    return xs, gam, bet, bias


def wl_rows(torch, kernels, op, rows=32768, cols=4096):
    from metalhlo_amd import _lib
    lib = _lib.load()
    xs, gam, bet, bias = _rows(torch, rows, cols)
    ys = [torch.empty_like(x) for x in xs]
    st = lambda: torch.cuda.current_stream().cuda_stream
    n = len(xs)
    base = 2.0 * rows * cols * 2
    if op == "softmax":
        fn = lambda i: lib.mhip_softmax(st(), xs[i % n].data_ptr(), ys[i % n].data_ptr(), rows, cols, 3)
        extra, kern = 0, "row_split_kernel<bf16,softmax>"
    elif op == "layer_norm":
        fn = lambda i: lib.mhip_layer_norm(st(), xs[i % n].data_ptr(), gam.data_ptr(), bet.data_ptr(),
                                           ys[i % n].data_ptr(), rows, cols, 1e-5, 3)
        extra, kern = 2 * cols * 2, "row_split_kernel<bf16,layer_norm>"
    elif op == "rms_norm":
        fn = lambda i: lib.mhip_rms_norm(st(), xs[i % n].data_ptr(), gam.data_ptr(), ys[i % n].data_ptr(),
                                         rows, cols, 1e-6, 3)
        extra, kern = cols * 2, "row_split_kernel<bf16,rms_norm>"
    elif op == "bias_gelu":
        fn = lambda i: lib.mhip_bias_gelu(st(), xs[i % n].data_ptr(), bias.data_ptr(), ys[i % n].data_ptr(),
                                          rows, cols, 3)
        extra, kern = cols * 2, "bias_gelu_tile_kernel<bf16>"
    else:
        raise ValueError(op)
    return dict(name=f"bf16 {op} [{rows},{cols}]", fn=fn, flops=0.0, bytes=base + extra, bound="hbm",
                kernel=kern)


def wl_copy(torch, kernels, nbytes=256 << 20):
    from metalhlo_amd import _lib
    lib = _lib.load()
    srcs = [torch.randint(0, 255, (nbytes,), dtype=torch.uint8, device="cuda") for _ in range(3)]
    dsts = [torch.empty_like(x) for x in srcs]
    st = lambda: torch.cuda.current_stream().cuda_stream
    return dict(name=f"device copy of {nbytes} bytes (calibration)",
                fn=lambda i: lib.mhip_copy(st(), srcs[i % 3].data_ptr(), dsts[i % 3].data_ptr(), nbytes),
                flops=0.0, bytes=2.0 * nbytes, bound="hbm", kernel="copy_kernel")


def wl_gpt2(torch, kernels, B=8, S=1024):
    from metalhlo_amd.gpt2 import GPT2, GPT2Config, init_params
    cfg = GPT2Config()
    model = GPT2(cfg, init_params(cfg, seed=5))
    import numpy as np
    ids = torch.from_numpy(np.random.default_rng(5).integers(0, cfg.vocab, (B, S)).astype(np.int32)).cuda()
    graphed = model.capture(ids)     # one HIP graph replay per step instead of ~135 host launches
    return dict(name=f"GPT-2-small forward B{B} S{S}, bf16 compute / fp32 params (converted every step), HIP graph replay",
                fn=lambda i: graphed(ids), flops=GPT2.flops(cfg, B, S), bytes=0.0, bound="mfma",
                kernel="fused pipeline (convert, embed, 12 x [LN, GEMM+bias, attention, GEMM+bias+residual, LN, "
                       "GEMM+bias+GELU, GEMM+bias+residual], LN, logits GEMM)")


def wl_gpt2_capi(torch, kernels, B=8, S=1024):
    """The same forward pass written as ONE plain StableHLO module (no custom calls, fp32
    parameters) and run through the C API: mhlo_compile recognises the fused operators,
    mhlo_execute runs them (optimisation level 3: replayed as one HIP graph that writes the logits
    into a buffer of their own).  Parameters stay resident as mhlo buffers; a step is one
    mhlo_execute (synchronous: it returns when the logits are complete) plus the release of
    its result.  Timed by the host clock around the calls."""
    import ctypes
    import numpy as np
    from metalhlo_amd import capi, programs
    from metalhlo_amd.gpt2 import GPT2, GPT2Config, init_params
    cfg = GPT2Config()
    text = programs.gpt2_program(B, S, cfg.n_layer, cfg.n_head, cfg.d_model // cfg.n_head, cfg.d_ff, cfg.vocab, cfg.n_pos)
    sess = capi.Session()
    exe = sess.compile(text, opt_level=3)      # O3: from the second execution on the op list is replayed as one HIP graph
    p = init_params(cfg, seed=5)
    rng = np.random.default_rng(5)
    ids = rng.integers(0, cfg.vocab, (B, S)).astype(np.int32)
    arrs = [(ids, "i32"), (p["wte"], "f32"), (p["wpe"], "f32")]
    for l in p["layers"]:
        arrs += [(l[n], "f32") for n in programs.GPT2_LAYER_PARAMS]
    arrs += [(p["lnf_g"], "f32"), (p["lnf_b"], "f32")]
    bufs = [sess.buffer(a, t) for a, t in arrs]
    arr = (ctypes.c_void_p * len(bufs))(*bufs)
    outs = (ctypes.c_void_p * 1)()
    got = ctypes.c_int32()

    def step(i):
        rc = sess.lib.mhlo_execute(exe, arr, len(bufs), outs, ctypes.byref(got))
        if rc != 0:
            raise RuntimeError("mhlo_execute failed: %s" % sess.lib.mhlo_get_last_error())
        sess.lib.mhlo_buffer_destroy(outs[0])
    return dict(name=f"GPT-2-small forward B{B} S{S} from one plain StableHLO module through mhlo_compile / mhlo_execute "
                     f"(fp32 parameters converted every step, {len(sess.ops(exe))} operations after pattern recognition)",
                fn=step, flops=GPT2.flops(cfg, B, S), bytes=0.0, bound="mfma", host_timed=True, keep=(sess, bufs),
                kernel="mhlo_execute (HIP graph replay): batched converts, embedding, 12 x 7 fused kernels, LN, logits GEMM")


def measure(wl, steps, warmup, torch, key=None):
    sampler = DeviceSampler() if wl["bound"] == "mfma" else None
    if sampler is not None and sampler.available():
        sampler.start()
    else:
        sampler = None
    t_begin = time.perf_counter()
    _ramp(wl["fn"], torch)
    sec, wall, each, (t0, t1) = _time_launches(wl["fn"], steps, warmup, torch)
    # power and clock: the samples of the second half of ramp + warm-up + timed launches (one kernel
    # throughout, so the steady state the timed launches run in)
    dev = sampler.stop(since=t_begin + 0.5 * (t1 - t_begin)) if sampler else None
    if wl.get("host_timed"):        # the calls are synchronous and run on the library's own stream
        sec = wall
    med, low = each[len(each) // 2], each[0]
    if wl["bound"] == "mfma":
        ach = wl["flops"] / sec / 1e12
        peak = wl.get("peak", PEAK_BF16_TFLOPS)
        roof = dict(bound="mfma", achieved=round(ach, 2), peak=peak, unit="TFLOP/s",
                    frac=round(ach / peak, 4), traffic=MEASURED_TRAFFIC.get(key))
        if dev:
            roof.update(power_w=dev["power_w"], power_cap_w=dev["power_cap_w"], clock_mhz=dev["clock_mhz"],
                        device_samples=dev["samples"])
            if dev["clock_mhz"]:
                # what the same cycles would give at the 2400 MHz the peak figure is quoted for
                roof["frac_at_clock"] = round(ach / peak * PEAK_CLOCK_MHZ / dev["clock_mhz"], 4)
        value, unit = ach, "TFLOP/s"
    else:
        ach = wl["bytes"] / sec / 1e9
        roof = dict(bound="hbm", achieved=round(ach, 1), peak=PEAK_HBM_GBS, unit="GB/s",
                    frac=round(ach / PEAK_HBM_GBS, 4), traffic=MEASURED_TRAFFIC.get(key))
        value, unit = ach, "GB/s"
    roof["traffic_commit"] = TRAFFIC_COMMIT if MEASURED_TRAFFIC.get(key) else None
    r = dict(workload=wl["name"], kernel=wl["kernel"], value=round(value, 2), unit=unit,
             us_per_launch=round(sec * 1e6, 2), wall_us_per_launch=round(wall * 1e6, 2), roofline=roof)
    if not wl.get("host_timed"):
        r.update(median_us=round(med * 1e6, 2), min_us=round(low * 1e6, 2))
    return r


# ---------------------------------------------------------------- shader clock under load
def clock_probe(torch, kernels, seconds=2.0):
    """The device lowers its shader clock when a kernel would exceed the board's power limit, and
    how far depends on the operand bits.  For the two matrix workloads: launches back to back for
    `seconds` while `rocm-smi --showclocks` is sampled from a second thread, once on the
    benchmark's random operands and once on zeros (which switch almost nothing and leave the
    clock at its maximum), then the time of 20 launches.  Prints one JSON object."""
    import re
    import subprocess
    import threading

    def sample(stop, out):
        # fallback where the hwmon files are not readable: the command-line tool, a few samples a second
        while not stop.is_set():
            r = subprocess.run(["/opt/rocm/bin/rocm-smi", "--showclocks", "--showpower"], capture_output=True, text=True)
            m = re.search(r"sclk clock level: \d+: \((\d+)Mhz\)", r.stdout)
            w = re.search(r"Power \(W\): ([0-9.]+)", r.stdout)
            if m:
                out.append((int(m.group(1)), float(w.group(1)) if w else None))
            time.sleep(0.2)

    def run(fn):
        hw = DeviceSampler()
        stop, smi = threading.Event(), []
        if hw.available():
            hw.start()
            th = None
        else:
            th = threading.Thread(target=sample, args=(stop, smi))
            th.start()
        t0 = time.time()
        t_half = time.perf_counter() + seconds / 2
        while time.time() - t0 < seconds:
            for _ in range(20):
                fn()
            torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(20):
            fn()
        e1.record()
        torch.cuda.synchronize()
        out = dict(us_per_launch=round(e0.elapsed_time(e1) / 20 * 1e3, 1))
        if th is None:
            d = hw.stop(since=t_half)
            out.update(sclk_mhz=d["clock_mhz"], power_w=d["power_w"], power_cap_w=d["power_cap_w"], source="hwmon")
        else:
            stop.set()
            th.join()
            tail = smi[len(smi) // 2:] or [(0, None)]
            ws = [w for _, w in tail if w is not None]
            out.update(sclk_mhz=round(sum(c for c, _ in tail) / len(tail)),
                       power_w=round(sum(ws) / len(ws), 1) if ws else None, source="rocm-smi")
        return out

    res = {}
    M = 4096
    g = torch.Generator(device="cuda").manual_seed(2)
    c = torch.empty(M, M, dtype=torch.bfloat16, device="cuda")
    for tag in ("uniform", "zeros"):
        if tag == "uniform":
            a = (torch.rand(M, M, generator=g, device="cuda") * 2 - 1).to(torch.bfloat16)
            b = (torch.rand(M, M, generator=g, device="cuda") * 2 - 1).to(torch.bfloat16)
        else:
            a = torch.zeros(M, M, dtype=torch.bfloat16, device="cuda")
            b = torch.zeros(M, M, dtype=torch.bfloat16, device="cuda")
        r = run(lambda: kernels.matmul(a, b, out=c))
        r["tflops"] = round(2.0 * M ** 3 / r["us_per_launch"] / 1e6, 1)
        res[f"gemm 4096^3 bf16, {tag} operands"] = r
    B, H, S, D = 4, 32, 4096, 128
    for tag in ("normal", "zeros"):
        if tag == "normal":
            q, k, v = (torch.randn(B, H, S, D, generator=g, device="cuda").to(torch.bfloat16) for _ in range(3))
        else:
            q, k, v = (torch.zeros(B, H, S, D, dtype=torch.bfloat16, device="cuda") for _ in range(3))
        r = run(lambda: kernels.flash_attention(q, k, v, is_causal=True))
        r["tflops"] = round(2.0 * B * H * S * S * D / r["us_per_launch"] / 1e6, 1)
        res[f"causal attention B4 H32 S4096 D128 bf16, {tag} operands"] = r
    x = torch.randn(32768, 4096, generator=g, device="cuda").to(torch.bfloat16)
    res["softmax [32768,4096] bf16"] = run(lambda: kernels.softmax(x))
    print(json.dumps({"clock_probe": res, "seconds_of_load_before_timing": seconds}))


# ---------------------------------------------------------------- CPU baselines
def _best_of(fn, reps=3):
    fn()                                    # warm-up
    best = float("inf")
    for _ in range(reps):
        t0 = time.perf_counter()
        fn()
        best = min(best, time.perf_counter() - t0)
    return best


def cpu_baseline_gemm_port(sample_rows=4096, N=4096, K=4096):
    """The C restatement of the oracle (OpenMP) on the same GEMM."""
    import numpy as np
    from oracle import oracle
    lib = C.CDLL(os.path.join(ROOT, "oracle", "liboracle.so"))
    lib.orc_num_threads.restype = C.c_int
    rng = np.random.default_rng(2)
    a = oracle.bf16_round_bits(rng.uniform(-1, 1, (sample_rows, K)).astype(np.float32))
    b = oracle.bf16_round_bits(rng.uniform(-1, 1, (K, N)).astype(np.float32))
    c = np.empty((sample_rows, N), np.uint16)
    p = lambda x: x.ctypes.data_as(C.c_void_p)
    args = (p(a), p(b), p(c), C.c_int64(sample_rows), C.c_int64(N), C.c_int64(K), 1)
    best = _best_of(lambda: lib.orc_gemm(*args))
    return dict(value=round(2.0 * sample_rows * N * K / best / 1e12, 5), unit="TFLOP/s",
                cores=int(lib.orc_num_threads()), kind="port",
                sample=f"oracle/oracle_kernels.c orc_gemm on {sample_rows} of 4096 rows of A "
                       f"(x full B), bf16 in / fp32 accumulate, one warm-up + best of 3 "
                       f"({best:.2f} s each); host has {os.cpu_count()} logical CPUs")


def cpu_baseline_torch(name, torch):
    """The operator of workload `name` with torch's CPU kernels (the library stand-in for the
    CPU path the reference's own suites compare with; jax is not installed), on a bounded
    sample, scaled to the workload's unit.  `cores` = torch's intra-op threads."""
    import torch.nn.functional as F
    th = torch.get_num_threads()
    g = torch.Generator().manual_seed(7)
    bf = torch.bfloat16
    base = dict(cores=th, kind="port")
    if name in ("gemm", "gemm_f32"):
        dt = bf if name == "gemm" else torch.float32
        a = (torch.rand(4096, 4096, generator=g) * 2 - 1).to(dt)
        b = (torch.rand(4096, 4096, generator=g) * 2 - 1).to(dt)
        t = _best_of(lambda: torch.matmul(a, b))
        return dict(base, value=round(2.0 * 4096 ** 3 / t / 1e12, 4), unit="TFLOP/s",
                    sample=f"torch.matmul on CPU, {'bf16' if name == 'gemm' else 'fp32'} 4096^3 (the whole workload), best of 3: {t:.3f} s")
    if name in ("attention", "attention_full", "attention_f32"):
        S, causal = (4096, True) if name == "attention" else (2048, name == "attention_f32")
        q, k, v = (torch.randn(1, 1, S, 128, generator=g).to(torch.float32 if name == "attention_f32" else bf) for _ in range(3))
        t = _best_of(lambda: F.scaled_dot_product_attention(q, k, v, is_causal=causal))
        flops = 4.0 * S * S * 128 * (0.5 if causal else 1.0)
        return dict(base, value=round(flops / t / 1e12, 4), unit="TFLOP/s",
                    sample=f"torch scaled_dot_product_attention on CPU, {'fp32' if name == 'attention_f32' else 'bf16'}, ONE of the 128 (batch, head) slices "
                           f"(S {S}, D 128, {'causal' if causal else 'full'}), best of 3: {t:.3f} s; the rate carries over, "
                           f"the whole workload is 128 such slices")
    if name in ("softmax", "layer_norm", "rms_norm", "bias_gelu"):
        rows, cols = 8192, 4096
        x = torch.randn(rows, cols, generator=g).to(bf)
        w = torch.ones(cols, dtype=bf)
        z = torch.zeros(cols, dtype=bf)
        fn = {"softmax": lambda: F.softmax(x, dim=-1),
              "layer_norm": lambda: F.layer_norm(x, (cols,), w, z, 1e-5),
              "rms_norm": lambda: (x.float() * torch.rsqrt(x.float().pow(2).mean(-1, keepdim=True) + 1e-6) * w.float()).to(bf),
              "bias_gelu": lambda: F.gelu(x + z, approximate="tanh")}[name]
        t = _best_of(fn)
        return dict(base, value=round(2.0 * rows * cols * 2 / t / 1e9, 2), unit="GB/s",
                    sample=f"torch on CPU, bf16, {rows} of the 32768 rows x {cols} (algorithmic bytes of the sample / time), "
                           f"best of 3: {t * 1e3:.1f} ms")
    if name in ("gpt2", "gpt2_capi"):
        from metalhlo_amd.gpt2 import GPT2Config, init_params
        cfg = GPT2Config()
        p = init_params(cfg, seed=5)
        tb = lambda a: torch.from_numpy(a).to(bf)
        wte, wpe = tb(p["wte"]), tb(p["wpe"])
        layers = [{k: tb(v) for k, v in l.items()} for l in p["layers"]]
        lnf = tb(p["lnf_g"]), tb(p["lnf_b"])
        ids = torch.randint(0, cfg.vocab, (1, 1024), generator=g)
        d, H = cfg.d_model, cfg.n_head

        def fwd():
            x = F.embedding(ids, wte) + wpe[None, :1024]
            for l in layers:
                h = F.layer_norm(x, (d,), l["ln1_g"], l["ln1_b"], 1e-5)
                q, k, v = F.linear(h, l["w_qkv"].T, l["b_qkv"]).split(d, dim=-1)
                sh = lambda t_: t_.view(1, 1024, H, d // H).transpose(1, 2)
                a = F.scaled_dot_product_attention(sh(q), sh(k), sh(v), is_causal=True).transpose(1, 2).reshape(1, 1024, d)
                x = x + F.linear(a, l["w_o"].T, l["b_o"])
                h = F.layer_norm(x, (d,), l["ln2_g"], l["ln2_b"], 1e-5)
                x = x + F.linear(F.gelu(F.linear(h, l["w_fc"].T, l["b_fc"]), approximate="tanh"), l["w_proj"].T, l["b_proj"])
            return F.linear(F.layer_norm(x, (d,), lnf[0], lnf[1], 1e-5), wte)
        with torch.no_grad():
            t = _best_of(fwd, reps=2)
        return dict(base, value=round(t * 8 * 1e3, 1), unit="ms",
                    sample=f"torch on CPU, bf16, ONE of the 8 sequences (12 layers, S 1024, full vocabulary): {t * 1e3:.0f} ms, "
                           f"times 8 for the batch")
    return None


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--workload", default="gemm",
                    choices=["gemm", "gemm_f32", "attention", "attention_full", "attention_f32", "softmax", "layer_norm", "rms_norm", "bias_gelu", "copy",
                             "gpt2", "gpt2_capi"])
    ap.add_argument("--ramp-ms", type=float, default=150.0,
                    help="milliseconds of untimed launches of the same kernel in front of the warm-up steps (0 = none)")
    ap.add_argument("--only", action="store_true", help="time only --workload (for profiling runs)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--clock-probe", action="store_true",
                    help="instead of the benchmark: shader clock and time per launch of the matrix workloads under "
                         "sustained load, on random and on all-zero operands")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on exactly one GPU (the reference is single-device and "
                 "every workload here shards without communication); use --gpus 1")

    import torch
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible; the kernels have no CPU path")
    global RAMP_MS
    RAMP_MS = args.ramp_ms
    from metalhlo_amd import _lib, kernels
    _lib.load()
    torch.cuda.set_device(0)
    if args.clock_probe:
        clock_probe(torch, kernels)
        return

    def build(name):
        if name == "gemm":
            return wl_gemm(torch, kernels)
        if name == "gemm_f32":
            return wl_gemm_f32(torch, kernels)
        if name == "attention":
            return wl_attention(torch, kernels, causal=True)
        if name == "attention_full":
            return wl_attention(torch, kernels, S=2048, causal=False)
        if name == "attention_f32":
            return wl_attention(torch, kernels, S=2048, causal=True, fp32=True)
        if name == "copy":
            return wl_copy(torch, kernels)
        if name == "gpt2":
            return wl_gpt2(torch, kernels)
        if name == "gpt2_capi":
            return wl_gpt2_capi(torch, kernels)
        return wl_rows(torch, kernels, name)

    slow = ("gpt2", "gpt2_capi")        # milliseconds per step: fewer steps

    def run(name):
        k = min(args.steps, 10) if name in slow else args.steps
        w = min(args.warmup, 3) if name in slow else args.warmup
        wl = build(name)
        r = measure(wl, k, w, torch, name)
        if name in slow:
            r["fwd_ms"] = round(r["us_per_launch"] / 1e3, 3)
        del wl
        torch.cuda.empty_cache()
        return r

    head = run(args.workload)
    others = {}
    if not args.only:
        for name in ["gemm", "gemm_f32", "attention", "attention_full", "attention_f32", "softmax", "layer_norm", "rms_norm", "bias_gelu",
                     "gpt2", "gpt2_capi"]:
            if name == args.workload:
                continue
            others[name] = run(name)
            print(f"[bench] {name}: {others[name]['value']} {others[name]['unit']} "
                  f"({others[name]['roofline']['frac'] * 100:.1f}% of peak)", file=sys.stderr, flush=True)
    cpu = None
    if not args.no_cpu:
        # the CPU leg: after every GPU measurement, on the host cores, bounded samples
        cpu = cpu_baseline_torch(args.workload, torch)
        if args.workload == "gemm" and cpu is not None:
            cpu["c_port"] = cpu_baseline_gemm_port()
        for name in others:
            others[name]["cpu_baseline"] = cpu_baseline_torch(name, torch)
            print(f"[bench] cpu {name}: {others[name]['cpu_baseline']['value']} {others[name]['cpu_baseline']['unit']}",
                  file=sys.stderr, flush=True)

    line = {
        "metric": "bf16 attn/GEMM TFLOP/s + norm/softmax GB/s (% roofline); GPT-2 fwd ms",
        "value": head["value"], "unit": head["unit"], "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(head["us_per_launch"] / 1e3, 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32" if args.workload.endswith("_f32") else "bf16", "data": "synthetic",
        "config": {"workload": head["workload"], "kernel": head["kernel"]},
        "clock_ramp_ms": args.ramp_ms,
        "roofline": head["roofline"],
        "cpu_baseline": cpu,
        "kernels": others,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
