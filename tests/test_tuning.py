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
        assert variant in ((128, 256, 2560, 2561) if tiles >= 192 else (128, 256, 2561)) and us > 0
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
