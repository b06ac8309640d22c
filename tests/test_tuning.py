"""Tuning table of the kernel library: text round trip (no GPU needed) and the tuning
passes for GEMM, the row operators and attention (GPU; the tuned launches are checked
against the float64 oracle, not against themselves)."""
import numpy as np
import pytest


def test_tuning_table_round_trip(lib, tmp_path):
    lib.mhip_tuning_clear()
    assert lib.mhip_tuning_count() == 0
    src = tmp_path / "in.txt"
    src.write_text("# comment\n"
                   "gemm gfx950/256 4096 4096 4096 1 0 0 3 = 2560 @ 108.5\n"
                   "gemm gfx942/304 4096 4096 4096 1 0 0 3 = 256 @ 150\n"          # another device: kept, never used
                   "row gfx950/256 1 3 32768 4096 1 1 = 2 2 1 0 @ 85.4\n"
                   "attention gfx950/256 3 128 4096 4096 128 1 = 3 @ 553.25\n")
    assert lib.mhip_tuning_load(str(src).encode()) == 0
    assert lib.mhip_tuning_count() == 4
    assert lib.mhip_tuning_load(str(src).encode()) == 0      # merging the same entries adds nothing
    assert lib.mhip_tuning_count() == 4
    dst = tmp_path / "out.txt"
    assert lib.mhip_tuning_save(str(dst).encode()) == 0
    lines = [l for l in dst.read_text().splitlines() if not l.startswith("#")]
    assert sorted(lines) == ["attention gfx950/256 3 128 4096 4096 128 1 = 3 @ 553.250",
                             "gemm gfx942/304 4096 4096 4096 1 0 0 3 = 256 @ 150.000",
                             "gemm gfx950/256 4096 4096 4096 1 0 0 3 = 2560 @ 108.500",
                             "row gfx950/256 1 3 32768 4096 1 1 = 2 2 1 0 @ 85.400"]
    for text in ("gemm gfx950/256 1 2 3 1 0 0 3 = 77 @ 1.0\n",            # 77 is no kernel variant
                 "row gfx950/256 1 3 8 8 1 1 = 3 1 1 0 @ 1.0\n",            # launch kind 3 does not exist
                 "attention gfx950/256 3 1 1 1 64 0 = 9 @ 1.0\n",
                 "conv gfx950/256 1 = 1 @ 1.0\n",                           # unknown operator
                 "gemm gfx950/256 1 2 3 1 0 0 3 2560 108.5\n"):             # the old, device-less form
        bad = tmp_path / "bad.txt"
        bad.write_text(text)
        assert lib.mhip_tuning_load(str(bad).encode()) == 1 and b"malformed" in lib.mhip_last_error(), text
    assert lib.mhip_tuning_load(str(tmp_path / "missing.txt").encode()) == 1
    assert lib.mhip_tuning_save(None) == 1
    lib.mhip_tuning_clear()
    assert lib.mhip_tuning_count() == 0
    assert lib.mhip_tuning_device()            # "nodevice/0" here, "<arch>/<compute units>" on a GPU


def _as64(t):
    return t.float().cpu().numpy().astype(np.float64)


def _close(got, exp, tol, what):
    e = np.abs(_as64(got) - exp)
    assert (e <= np.maximum(tol, tol * np.abs(exp))).all(), what


@pytest.mark.gpu
def test_gemm_autotune_picks_a_valid_variant_and_keeps_results():
    import torch
    from metalhlo_amd import kernels
    from oracle import oracle
    kernels.tuning_clear()
    torch.manual_seed(3)
    for (M, N, K, tb) in [(4096, 4096, 1024, False), (1024, 768, 768, False), (4096, 2048, 2048, True)]:
        a = (torch.rand(M, K, device="cuda") * 2 - 1).bfloat16()
        b = (torch.rand((N, K) if tb else (K, N), device="cuda") * 2 - 1).bfloat16()
        before = kernels.matmul(a, b, trans_b=tb)
        variant, us = kernels.autotune_matmul(a, b, trans_b=tb, iters=5)
        tiles = ((M + 255) // 256) * ((N + 255) // 256)
        ring = (2560, 2561, 2562, 2563, 2564, 2565, 2566, 2567, 2568, 2569, 2570)      # the generated family, streamed tiles, the column split
        assert variant in ((128, 256) + ring if tiles >= 192 else (128, 256, 2561, 2564, 2565, 2568, 2569)) and us > 0
        tuned = kernels.matmul(a, b, trans_b=tb)
        # the tuned launch against the oracle on sampled rows ...
        rows = [0, 1, M // 2, M - 1]
        exp = oracle.gemm(_as64(a[rows]), _as64(b), trans_b=tb)
        _close(tuned[rows], exp, 2e-2, f"tuned GEMM {M}x{N}x{K}")
        # ... and every variant accumulates in the same order: the choice changes speed, not bits
        assert torch.equal(tuned, before)
    assert kernels.tuning_count() == 3
    with pytest.raises(Exception):
        kernels.autotune_matmul(a.float(), b.float())
    kernels.tuning_clear()


@pytest.mark.gpu
@pytest.mark.parametrize("op", ["softmax", "layer_norm", "rms_norm"])
def test_row_autotune_result_is_used_and_matches_the_oracle(op, tmp_path):
    import torch
    from metalhlo_amd import kernels
    from oracle import oracle
    kernels.tuning_clear()
    rng = np.random.default_rng(5)
    for rows, cols, dt, tol in [(2048, 4096, torch.bfloat16, 2e-2), (4096, 768, torch.bfloat16, 2e-2), (512, 1024, torch.float32, 1e-5)]:
        x = torch.from_numpy((rng.standard_normal((rows, cols)) * 2 + 0.5).astype(np.float32)).to(dt).cuda()
        g = torch.from_numpy((1 + 0.1 * rng.standard_normal(cols)).astype(np.float32)).to(dt).cuda()
        b = torch.from_numpy((0.1 * rng.standard_normal(cols)).astype(np.float32)).to(dt).cuda()
        args = {"softmax": (), "layer_norm": (g, b), "rms_norm": (g,)}[op]
        choice, us = kernels.autotune_row(op, x, *args, eps=1e-5, iters=5)
        assert choice[0] in (1, 2) and choice[1] in (1, 2) and choice[2] in (0, 1) and 0 <= choice[3] <= 16 and us > 0
        got = {"softmax": lambda: kernels.softmax(x), "layer_norm": lambda: kernels.layer_norm(x, g, b, eps=1e-5),
               "rms_norm": lambda: kernels.rms_norm(x, g, eps=1e-5)}[op]()
        exp = {"softmax": lambda: oracle.softmax(_as64(x)), "layer_norm": lambda: oracle.layer_norm(_as64(x), _as64(g), _as64(b), 1e-5),
               "rms_norm": lambda: oracle.rms_norm(_as64(x), _as64(g), 1e-5)}[op]()
        _close(got, exp, tol, f"tuned {op} [{rows},{cols}] {dt} as {choice}")
    assert kernels.tuning_count() == 3
    # the table names this device; saved and loaded again it still serves the same problems
    path = tmp_path / "t.txt"
    kernels.tuning_save(path)
    text = path.read_text()
    assert text.count(f"row {kernels.tuning_device()} ") == 3 and kernels.tuning_device().startswith("gfx")
    kernels.tuning_clear()
    kernels.tuning_load(path)
    assert kernels.tuning_count() == 3
    kernels.tuning_clear()


@pytest.mark.gpu
@pytest.mark.parametrize("causal", [False, True])
def test_attention_autotune_matches_the_oracle(causal):
    import torch
    from metalhlo_amd import kernels
    from oracle import oracle
    kernels.tuning_clear()
    rng = np.random.default_rng(6)
    for B, H, S, D in [(1, 2, 512, 128), (2, 2, 320, 64)]:
        q, k, v = (torch.from_numpy(rng.standard_normal((B, H, S, D)).astype(np.float32)).bfloat16().cuda() for _ in range(3))
        variant, us = kernels.autotune_attention(q, k, v, is_causal=causal, iters=3)
        assert variant in ((1, 2, 3) if D == 128 and causal else (1, 2) if D == 128 else (1,)) and us > 0
        got = kernels.flash_attention(q, k, v, is_causal=causal)
        exp = oracle.attention(_as64(q), _as64(k), _as64(v), is_causal=causal)
        _close(got, exp, 2e-2, f"tuned attention B{B} H{H} S{S} D{D} as variant {variant}")
        # each variant on its own, forced through the table, against the same oracle
    assert kernels.tuning_count() == 2
    kernels.tuning_clear()


@pytest.mark.gpu
def test_gemm_autotune_in_model_and_the_shipped_table(lib, tmp_path):
    """The in-model pass (caches emptied and A rewritten before every timed launch) records a valid
    variant, and a table entry really moves the choice: for a GEMM of the GPT-2 forward pass the
    heuristic's variant and a different variant named by a loaded table are both observed through
    mhip_gemm_last_variant, with bit-identical results.  The table that ships with the library (when
    there is one for this device) parses, names this device and only variants that exist."""
    import ctypes as C
    import os
    import torch
    from metalhlo_amd import kernels
    kernels.tuning_clear()
    torch.manual_seed(4)
    M, N, K = 8192, 768, 768                                    # the attention output projection of GPT-2-small B8 S1024
    a = (torch.rand(M, K, device="cuda") * 2 - 1).bfloat16()
    b = ((torch.rand(K, N, device="cuda") * 2 - 1) * K ** -0.5).bfloat16()
    plain = kernels.matmul(a, b)
    default_variant = lib.mhip_gemm_last_variant()
    assert default_variant in (128, 256, 2560, 2561, 2563, 2567, 2569)      # what the heuristic can choose
    other = 2564 if default_variant != 2564 else 2561
    table = tmp_path / "t.txt"
    table.write_text(f"gemm {kernels.tuning_device()} {M} {N} {K} 1 0 0 3 = {other} @ 1.0\n")
    kernels.tuning_load(table)
    tuned = kernels.matmul(a, b)
    assert lib.mhip_gemm_last_variant() == other
    assert torch.equal(tuned, plain)
    kernels.tuning_clear()
    kernels.matmul(a, b)
    assert lib.mhip_gemm_last_variant() == default_variant
    # the in-model pass
    flush = torch.empty(512 << 20, dtype=torch.uint8, device="cuda")
    c = torch.empty(M, N, dtype=torch.bfloat16, device="cuda")
    var, us = C.c_int(), C.c_float()
    st = torch.cuda.current_stream().cuda_stream
    assert lib.mhip_gemm_autotune_in_model(st, a.data_ptr(), b.data_ptr(), None, c.data_ptr(), M, N, K, 1, 0, 0, 0, 0, 0, 0, 3, 5,
                                           flush.data_ptr(), flush.numel(), C.byref(var), C.byref(us)) == 0, lib.mhip_last_error()
    assert var.value in (128, 256, 2561, 2564, 2565, 2568, 2569) and us.value > 0 and kernels.tuning_count() == 1
    assert torch.equal(kernels.matmul(a, b), plain) and lib.mhip_gemm_last_variant() == var.value
    assert torch.equal(a, a.clone())                             # (A was rewritten in place with its own values)
    assert lib.mhip_gemm_autotune_in_model(st, a.data_ptr(), b.data_ptr(), None, c.data_ptr(), M, N, K, 1, 0, 0, 0, 0, 0, 0, 3, 5,
                                           flush.data_ptr(), 1 << 20, C.byref(var), C.byref(us)) == 1      # flush buffer too small
    kernels.tuning_clear()
    shipped = kernels.shipped_tuning_table()
    if os.path.exists(shipped):
        kernels.tuning_load(shipped)
        assert kernels.tuning_count() >= 5
        text = open(shipped).read()
        assert f"gemm {kernels.tuning_device()} 4096 4096 4096 1 0 0 3 = " in text
        assert f"attention {kernels.tuning_device()} 3 128 4096 4096 128 1 = " in text
        kernels.tuning_clear()
