"""Tuning table of the kernel library: text round trip (no GPU needed) and the GEMM
autotuner (GPU)."""
import ctypes as C

import pytest


def test_tuning_table_round_trip(lib, tmp_path):
    lib.mhip_tuning_clear()
    assert lib.mhip_tuning_count() == 0
    src = tmp_path / "in.txt"
    src.write_text("# comment\ngemm 4096 4096 4096 1 0 0 3 2560 108.5\ngemm 8192 768 768 1 0 0 3 128 21.0\n"
                   "gemm 8192 50257 768 1 0 1 3 256 984.25\n")
    assert lib.mhip_tuning_load(str(src).encode()) == 0
    assert lib.mhip_tuning_count() == 3
    assert lib.mhip_tuning_load(str(src).encode()) == 0      # merging the same entries adds nothing
    assert lib.mhip_tuning_count() == 3
    dst = tmp_path / "out.txt"
    assert lib.mhip_tuning_save(str(dst).encode()) == 0
    lines = [l for l in dst.read_text().splitlines() if not l.startswith("#")]
    assert sorted(lines) == ["gemm 4096 4096 4096 1 0 0 3 2560 108.500", "gemm 8192 50257 768 1 0 1 3 256 984.250",
                             "gemm 8192 768 768 1 0 0 3 128 21.000"]
    bad = tmp_path / "bad.txt"
    bad.write_text("gemm 1 2 3 1 0 0 3 77 1.0\n")            # 77 is no kernel variant
    assert lib.mhip_tuning_load(str(bad).encode()) == 1 and b"malformed" in lib.mhip_last_error()
    assert lib.mhip_tuning_load(str(tmp_path / "missing.txt").encode()) == 1
    assert lib.mhip_tuning_save(None) == 1
    lib.mhip_tuning_clear()
    assert lib.mhip_tuning_count() == 0


@pytest.mark.gpu
def test_gemm_autotune_picks_a_valid_variant_and_keeps_results():
    import torch
    from metalhlo_amd import kernels
    kernels.tuning_clear()
    torch.manual_seed(3)
    for (M, N, K, tb) in [(4096, 4096, 1024, False), (1024, 768, 768, False), (4096, 2048, 2048, True)]:
        a = (torch.rand(M, K, device="cuda") * 2 - 1).bfloat16()
        b = (torch.rand((N, K) if tb else (K, N), device="cuda") * 2 - 1).bfloat16()
        before = kernels.matmul(a, b, trans_b=tb)
        variant, us = kernels.autotune_matmul(a, b, trans_b=tb, iters=5)
        tiles = ((M + 255) // 256) * ((N + 255) // 256)
        assert variant in ((128, 256, 2560, 2561) if tiles >= 192 else (128, 256, 2561)) and us > 0
        # every variant accumulates in the same order: the tuned choice changes speed, not bits
        assert torch.equal(kernels.matmul(a, b, trans_b=tb), before)
    assert kernels.tuning_count() == 3
    with pytest.raises(Exception):
        kernels.autotune_matmul(a.float(), b.float())
    kernels.tuning_clear()
