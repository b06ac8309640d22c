"""Writes the tuning table that ships with the library for the device it runs on.

    python -m metalhlo_amd.tune [--out FILE] [--iters N]

Times, on the GPU in use, every kernel variant the library has for the problems of the benchmark
configurations and of the GPT-2-small forward pass (B8 S1024), keeps the fastest of each, and saves the
table as metalhlo_amd/tuning/<arch>_<compute units>.txt, which the kernel library loads at first use
on such a device.  The role of the reference's AutoTuner + TuningDatabase
(Sources/MetalHLOCore/Tuning/AutoTuner.swift:301-458, TuningDatabase.swift:109-150), with two
differences: the candidates are real kernels, and the GEMMs of the model are timed by the model
itself -- one shape at a time, each variant the shape can run, with the whole captured forward pass as
the clock -- because a GEMM in a loop of its own finds its operands in the caches and a GEMM in a
model does not, which changes which tile width and ring depth wins.  torch supplies device memory
and the stream only."""
from __future__ import annotations

import argparse
import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))

# GEMMs timed in a loop of their own, the benchmark's protocol: (M, N, K, trans_b)
LOOP_GEMMS = [(4096, 4096, 4096, 0)]
# GEMMs of the GPT-2-small forward pass (B8 S1024), timed INSIDE that pass: (name, M, N, K, trans_b)
MODEL_GEMMS = [
    ("QKV projection", 8192, 2304, 768, 0),
    ("attention output projection", 8192, 768, 768, 0),
    ("FFN up + GELU", 8192, 3072, 768, 0),
    ("FFN down", 8192, 768, 3072, 0),
    ("logits (tied embedding, rows padded to a multiple of 64)", 8192, 50304, 768, 1),
]
# the logits GEMM as the program from text writes it (N = 50257): timed on its own, caches emptied
TEXT_LOGITS = (8192, 50257, 768, 1)
GEMM_VARIANTS = [128, 256, 2560, 2561, 2562, 2563, 2564, 2565, 2566, 2567, 2568, 2569, 2570]
ATTENTION = [(4, 32, 4096, 128, 1), (4, 32, 2048, 128, 0)]            # B, H, S, D, causal
# operator (0 softmax, 1 LayerNorm, 2 RMSNorm), rows, cols.  Only the benchmark shapes: a row kernel between two
# GEMMs of a model is not timed in a loop of its own -- there the launch form decides which XCD's L2 holds
# the rows for the next kernel, and the form that wins alone (a persistent grid for [8192, 768]: 6.7 us)
# cost the GPT-2 pass 0.25 ms (LayerNorm 6.7 -> 9.6 us each, and every GEMM behind one 10 % slower).
ROWS = [(op, 32768, 4096) for op in (0, 1, 2)]


def _forward_us(model, ids, torch, replays=12):
    """Median microseconds of one replay of the captured forward pass."""
    graphed = model.capture(ids)
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(replays + 1)]
    for _ in range(3):
        graphed(ids)
    ev[0].record()
    for i in range(replays):
        graphed(ids)
        ev[i + 1].record()
    torch.cuda.synchronize()
    t = sorted(ev[i].elapsed_time(ev[i + 1]) * 1e3 for i in range(replays))
    del graphed
    torch.cuda.empty_cache()
    return t[replays // 2]


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--out", default=None)
    ap.add_argument("--iters", type=int, default=30)
    args = ap.parse_args()
    import numpy as np
    import torch
    from metalhlo_amd import _lib
    from metalhlo_amd.gpt2 import GPT2, GPT2Config, init_params
    lib = _lib.load()
    if not torch.cuda.is_available():
        raise SystemExit("tune: no GPU visible")
    lib.mhip_tuning_clear()                        # start from the heuristics, not from an older table
    dev = lib.mhip_tuning_device().decode()
    out = args.out or os.path.join(HERE, "tuning", dev.replace("/", "_") + ".txt")
    st = torch.cuda.current_stream().cuda_stream
    bf = torch.bfloat16
    var, us = C.c_int(), C.c_float()

    def check(rc, what):
        if rc != 0:
            raise SystemExit(f"tune: {what} failed: {lib.mhip_last_error().decode()}")

    def operands(M, N, K, tb):
        a = (torch.rand(M, K, device="cuda") * 2 - 1).to(bf)
        b = ((torch.rand((N, K) if tb else (K, N), device="cuda") * 2 - 1) * K ** -0.5).to(bf)
        return a, b, torch.empty(M, N, dtype=bf, device="cuda")

    for M, N, K, tb in LOOP_GEMMS:
        a, b, c = operands(M, N, K, tb)
        check(lib.mhip_gemm_autotune(st, a.data_ptr(), b.data_ptr(), None, c.data_ptr(), M, N, K, 1, 0, 0, 0, 0, tb, 0, 3,
                                     args.iters, C.byref(var), C.byref(us)), "gemm")
        print(f"gemm [{M},{K}] x [{K},{N}] in a loop: variant {var.value}, {us.value:.1f} us", flush=True)
        del a, b, c

    # ---- the GEMMs of the model, timed by the model: one shape at a time, every variant the shape can
    # run, the whole forward pass (a captured graph, replayed) as the clock
    cfg = GPT2Config()
    model = GPT2(cfg, init_params(cfg, seed=5))
    ids = torch.from_numpy(np.random.default_rng(5).integers(0, cfg.vocab, (8, 1024)).astype(np.int32)).cuda()
    base = _forward_us(model, ids, torch)
    print(f"GPT-2-small forward B8 S1024 on the heuristics: {base:.1f} us", flush=True)
    for name, M, N, K, tb in MODEL_GEMMS:
        best_v, best_t = 0, base
        for v in GEMM_VARIANTS:
            check(lib.mhip_tuning_set_gemm(M, N, K, 1, 0, tb, 3, v, 0.0), "set")
            t = _forward_us(model, ids, torch)
            print(f"  {name} [{M},{K}] x [{K},{N}] as variant {v}: forward {t:.1f} us", flush=True)
            if t < best_t * 0.995:              # a candidate must beat the incumbent by more than the noise (+-0.3 % from run to run)
                best_v, best_t = v, t
        check(lib.mhip_tuning_set_gemm(M, N, K, 1, 0, tb, 3, best_v, best_t), "set")
        print(f"{name}: " + (f"variant {best_v}, forward {best_t:.1f} us" if best_v else "the heuristic's choice stays"), flush=True)
        base = best_t
    del model
    torch.cuda.empty_cache()

    M, N, K, tb = TEXT_LOGITS
    a, b, c = operands(M, N, K, tb)
    flush = torch.empty(96 << 20, dtype=torch.uint8, device="cuda")
    check(lib.mhip_gemm_autotune_in_model(st, a.data_ptr(), b.data_ptr(), None, c.data_ptr(), M, N, K, 1, 0, 0, 0, 0, tb, 0, 3, 9,
                                          flush.data_ptr(), flush.numel(), C.byref(var), C.byref(us)), "gemm (caches emptied)")
    print(f"gemm [{M},{K}] x [{K},{N}] (B stored [N,K]), L2s emptied before each launch: variant {var.value}, {us.value:.1f} us", flush=True)
    del a, b, c, flush

    for B, H, S, D, causal in ATTENTION:
        q, k, v = (torch.randn(B, H, S, D, device="cuda").to(bf) for _ in range(3))
        o = torch.empty_like(q)
        check(lib.mhip_attention_autotune(st, q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), B, H, S, S, D, D ** -0.5,
                                          causal, 3, 10, C.byref(var), C.byref(us)), "attention")
        print(f"attention B{B} H{H} S{S} D{D} {'causal' if causal else 'full'}: variant {var.value}, {us.value:.1f} us", flush=True)
        del q, k, v, o
    choice = (C.c_int * 4)()
    for op, rows, cols in ROWS:
        x = torch.randn(rows, cols, device="cuda").to(bf)
        y = torch.empty_like(x)
        g = torch.ones(cols, dtype=bf, device="cuda")
        z = torch.zeros(cols, dtype=bf, device="cuda")
        check(lib.mhip_row_autotune(st, op, x.data_ptr(), g.data_ptr(), z.data_ptr(), y.data_ptr(), rows, cols, 1e-5, 3,
                                    args.iters, choice, C.byref(us)), "row operator")
        print(f"row operator {op} [{rows},{cols}]: {list(choice)}, {us.value:.1f} us", flush=True)
        del x, y
    torch.cuda.synchronize()
    os.makedirs(os.path.dirname(os.path.abspath(out)), exist_ok=True)
    check(lib.mhip_tuning_save(out.encode()), "save")
    print(f"{lib.mhip_tuning_count()} entries for {dev} -> {out}")


if __name__ == "__main__":
    main()
