"""GPU parity: dot_general GEMM through the C-ABI vs the float64 oracle on the
same (already rounded) operands.  bf16/fp16: 2e-2 relative; fp32: 1e-5 relative,
both with the floor max(tol, tol*|e|).  Integer-valued operands whose partial
sums are exactly representable must come out bit-exact."""
import json
import os

import numpy as np
import pytest
import torch

from oracle import oracle
from tests.util import NAME, TOL, as_f64, assert_close, to_dev

pytestmark = pytest.mark.gpu


def _ab(M, N, K, dtype, seed, ta=False, tb=False, batch=()):
    rng = np.random.default_rng(seed)
    a = rng.uniform(-1, 1, batch + ((K, M) if ta else (M, K)))
    b = rng.uniform(-1, 1, batch + ((N, K) if tb else (K, N)))
    return to_dev(a, dtype), to_dev(b, dtype)


# MFMA path: full tiles, ragged M/N/K (K tail not a multiple of 64), small-tile config
SHAPES16 = [(256, 256, 256), (512, 768, 128), (300, 520, 136), (64, 8, 8), (1, 8, 64),
            (1000, 264, 72), (2048, 2048, 512)]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=lambda d: NAME[d])
@pytest.mark.parametrize("layout", [(False, False), (False, True), (True, False), (True, True)],
                         ids=["nn", "nt", "tn", "tt"])
@pytest.mark.parametrize("shape", SHAPES16, ids=lambda s: "x".join(map(str, s)))
def test_gemm_16bit(shape, layout, dtype):
    from metalhlo_amd import kernels
    M, N, K = shape
    ta, tb = layout
    a, b = _ab(M, N, K, dtype, 21, ta, tb)
    c = kernels.matmul(a, b, trans_a=ta, trans_b=tb)
    assert c.shape == (M, N)
    assert_close(c, oracle.gemm(as_f64(a), as_f64(b), ta, tb), TOL[dtype], f"gemm {shape} {layout}")


@pytest.mark.parametrize("shape", [(4, 4, 4), (33, 17, 9), (64, 64, 64), (130, 70, 50)],
                         ids=lambda s: "x".join(map(str, s)))
def test_gemm_f32(shape):
    # fp32 accumulation error grows like sqrt(K)*2^-24*|a||b|; these K keep it
    # inside the reference's 1e-5 rule for uniform[-1,1] operands.
    from metalhlo_amd import kernels
    M, N, K = shape
    for ta, tb in [(False, False), (True, True)]:
        a, b = _ab(M, N, K, torch.float32, 22, ta, tb)
        c = kernels.matmul(a, b, trans_a=ta, trans_b=tb)
        assert_close(c, oracle.gemm(as_f64(a), as_f64(b), ta, tb), 1e-5, f"gemm f32 {shape}")


@pytest.mark.parametrize("layout", [(False, False), (False, True), (True, False), (True, True)], ids=["nn", "nt", "tn", "tt"])
@pytest.mark.parametrize("shape", [(128, 128, 64), (256, 384, 128), (300, 200, 72), (130, 70, 50), (64, 65, 17), (1000, 136, 256)],
                         ids=lambda s: "x".join(map(str, s)))
def test_gemm_f32_matrix_cores(shape, layout):
    """fp32 operands on v_mfma_f32_32x32x2_f32 (128x128 tiles): every layout, ragged M / N / K, leading
    dimensions that are no multiple of 4 (scalar staging), bias + activation + residual."""
    from metalhlo_amd import kernels
    M, N, K = shape
    ta, tb = layout
    a, b = _ab(M, N, K, torch.float32, 41, ta, tb)
    c = kernels.matmul(a, b, trans_a=ta, trans_b=tb)
    assert_close(c, oracle.gemm(as_f64(a), as_f64(b), ta, tb), 1e-5, f"gemm f32 mfma {shape} {layout}")
    rng = np.random.default_rng(42)
    bias = to_dev(rng.standard_normal(N), torch.float32)
    r = to_dev(rng.standard_normal((M, N)), torch.float32)
    y = kernels.matmul(a, b, bias=bias, activation="gelu", trans_a=ta, trans_b=tb, residual=r)
    exp = oracle.matmul_bias_act(as_f64(a), as_f64(b), as_f64(bias), "gelu", ta, tb) + as_f64(r)
    assert_close(y, exp, 1e-5, f"gemm f32 mfma epilogue {shape} {layout}")


def test_gemm_f32_matrix_cores_long_k_and_batch():
    """K = 4096: the rounding of a 4096-term fp32 sum exceeds 1e-5 of a result that happens to be
    small, for any summation order; the bound that holds is the forward error bound of a dot
    product, |c - c_exact| <= 1e-5 (|a| . |b|) -- still five digits of every product.  Also a batched
    problem, and the matrix-core kernel against the plain fp32 kernel."""
    import os
    from metalhlo_amd import kernels
    a, b = _ab(512, 384, 4096, torch.float32, 43)
    c = as_f64(kernels.matmul(a, b))
    A, B = as_f64(a), as_f64(b)
    assert np.all(np.abs(c - A @ B) <= 1e-5 * (np.abs(A) @ np.abs(B)))
    a, b = _ab(200, 136, 96, torch.float32, 44, batch=(3,))
    c = kernels.matmul(a, b)
    assert_close(c, oracle.gemm(as_f64(a), as_f64(b)), 1e-5, "batched f32")
    os.environ["MHIP_GEMM_F32_MFMA"] = "2"
    try:
        plain = kernels.matmul(a, b)
    finally:
        del os.environ["MHIP_GEMM_F32_MFMA"]
    assert_close(plain, as_f64(c), 1e-5, "plain vs matrix-core fp32 kernel")


def test_gemm_unaligned_falls_back():
    """K or N not a multiple of 8 (e.g. vocab 50257) cannot use 16-byte loads."""
    from metalhlo_amd import kernels
    a, b = _ab(40, 50257 // 100, 100, torch.bfloat16, 23)          # N = 502
    assert_close(kernels.matmul(a, b), oracle.gemm(as_f64(a), as_f64(b)), 2e-2, "N=502")
    a, b = _ab(40, 64, 100 + 3, torch.bfloat16, 24)                # K = 103
    assert_close(kernels.matmul(a, b), oracle.gemm(as_f64(a), as_f64(b)), 2e-2, "K=103")
    # tied output head: x [T,768] . wte[50257,768]^T — k-contiguous, MFMA path, odd N
    a, b = _ab(128, 50257, 768, torch.bfloat16, 25, tb=True)
    assert_close(kernels.matmul(a, b, trans_b=True), oracle.gemm(as_f64(a), as_f64(b), False, True),
                 2e-2, "logits")


def test_gemm_exact_small_integers():
    """Entries in {-2..2}: every product and partial sum is an integer far below
    2^24, and |C| <= 4K = 256 is exact in bf16 -> result must be bit-exact."""
    from metalhlo_amd import kernels
    rng = np.random.default_rng(26)
    M, N, K = 512, 384, 64
    a = rng.integers(-2, 3, (M, K)).astype(np.float64)
    b = rng.integers(-2, 3, (K, N)).astype(np.float64)
    for dtype in (torch.bfloat16, torch.float16):
        c = kernels.matmul(to_dev(a, dtype), to_dev(b, dtype))
        assert np.array_equal(as_f64(c), a @ b)
    # identity and all-ones closed forms
    eye = to_dev(np.eye(256), torch.bfloat16)
    x, _ = _ab(256, 256, 256, torch.bfloat16, 27)
    assert torch.equal(kernels.matmul(x, eye), x)
    assert torch.equal(kernels.matmul(eye, x), x)
    ones = to_dev(np.ones((256, 256)), torch.bfloat16)
    assert np.array_equal(as_f64(kernels.matmul(ones, ones)), np.full((256, 256), 256.0))


def test_gemm_batched_bias_activation():
    from metalhlo_amd import kernels
    rng = np.random.default_rng(28)
    a, b = _ab(96, 136, 72, torch.bfloat16, 29, batch=(5,))
    c = kernels.matmul(a, b)
    assert c.shape == (5, 96, 136)
    assert_close(c, oracle.gemm(as_f64(a), as_f64(b)), 2e-2, "batched")
    x, w = _ab(200, 264, 128, torch.bfloat16, 30)
    bias = to_dev(rng.standard_normal(264) * 0.5, torch.bfloat16)
    for act in ("none", "relu", "gelu", "silu", "tanh", "sigmoid", "gelu_exact"):
        y = kernels.matmul(x, w, bias=bias, activation=act)
        assert_close(y, oracle.matmul_bias_act(as_f64(x), as_f64(w), as_f64(bias), act), 2e-2, act)
    xf, wf = _ab(20, 24, 16, torch.float32, 31)
    bf = to_dev(rng.standard_normal(24), torch.float32)
    assert_close(kernels.matmul(xf, wf, bias=bf, activation="gelu"),
                 oracle.matmul_bias_act(as_f64(xf), as_f64(wf), as_f64(bf), "gelu"), 1e-5, "f32 gelu")


def test_reference_dot_known_answers():
    from metalhlo_amd import kernels
    kat = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "kat.json")))
    for case in kat["dot"]:
        lhs, rhs = np.array(case["lhs"], dtype=np.float64), np.array(case["rhs"], dtype=np.float64)
        lb, rb, lc, rc = (case[k] for k in ("lhs_batch", "rhs_batch", "lhs_contract", "rhs_contract"))
        # canonicalise exactly like the host does: batch dims first, contracting last/first
        lf = [i for i in range(lhs.ndim) if i not in lb and i not in lc]
        rf = [i for i in range(rhs.ndim) if i not in rb and i not in rc]
        a = np.transpose(lhs, lb + lf + lc)
        b = np.transpose(rhs, rb + rc + rf)
        bs = [lhs.shape[i] for i in lb]
        B = int(np.prod(bs)) if bs else 1
        M = int(np.prod([lhs.shape[i] for i in lf])) if lf else 1
        K = int(np.prod([lhs.shape[i] for i in lc])) if lc else 1
        N = int(np.prod([rhs.shape[i] for i in rf])) if rf else 1
        c = kernels.matmul(to_dev(a.reshape(B, M, K), torch.float32), to_dev(b.reshape(B, K, N), torch.float32))
        exp = np.array(case["y"], dtype=np.float64)
        got = as_f64(c).reshape(exp.shape)
        if case["tol"] == 0:
            assert np.array_equal(got, exp), case["src"]
        else:
            assert np.all(np.abs(got - exp) <= case["tol"]), case["src"]


def test_gemm_4096_sampled_rows():
    """The benchmark GEMM: 4096^3 bf16, uniform[-1,1] (seed 2). Oracle on 64 sampled rows."""
    from metalhlo_amd import kernels
    rng = np.random.default_rng(2)
    a = to_dev(rng.uniform(-1, 1, (4096, 4096)), torch.bfloat16)
    b = to_dev(rng.uniform(-1, 1, (4096, 4096)), torch.bfloat16)
    c = kernels.matmul(a, b)
    rows = np.r_[0, 1, 31, 32, 255, 256, 4095, rng.integers(0, 4096, 57)]
    exp = as_f64(a[rows]) @ as_f64(b)
    assert_close(c[rows], exp, 2e-2, "gemm 4096 sampled rows")
    # linearity in A: (2A).B == 2(A.B) exactly (power-of-two scaling commutes with rounding)
    assert torch.equal(kernels.matmul(a * 2, b), c * 2)


# Shapes with >= 192 tiles of 256x256 for the four-wave kernel with the hand-scheduled
# main loop (K stages of 32: a single stage, exits at several positions of the unrolled
# ring of ten stages, more than one trip through it, ragged M / N, every operand layout).
BIG = [(4096, 3072, 32), (3585, 3848, 96), (4000, 3608, 160), (3600, 4104, 448), (8192, 2304, 768),
       (4096, 4096, 1056)]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=lambda d: NAME[d])
@pytest.mark.parametrize("layout", [(False, False), (False, True), (True, False), (True, True)],
                         ids=["nn", "nt", "tn", "tt"])
@pytest.mark.parametrize("shape", BIG, ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("tile", ["2560", "2561", "2564", "2565", "2566", "2568"],
                         ids=["256x256", "256x128", "256x128-ring6", "256x128-ring4", "256x256-ring4", "256x128-two-per-cu"])
def test_gemm_large_tiles(shape, layout, dtype, tile, lib):
    """The four-wave ring kernel in every member of its generated family (tile width x ring depth;
    forced: also where the default picks another kernel), ragged M and N included."""
    from metalhlo_amd import kernels
    M, N, K = shape
    ta, tb = layout
    a, b = _ab(M, N, K, dtype, 27, ta, tb)
    rng = np.random.default_rng(28)
    bias = to_dev(rng.standard_normal(N) * 0.5, dtype)
    os.environ["MHIP_GEMM_TILE"] = tile
    try:
        c = kernels.matmul(a, b, bias, "relu", trans_a=ta, trans_b=tb)
        # (operand rows that are not 16-byte aligned -- a transposed A with odd M -- run the scalar kernel)
        aligned = (not ta or M % 8 == 0) and (tb or N % 8 == 0)
        assert lib.mhip_gemm_last_variant() == (int(tile) if aligned else 0)
    finally:
        del os.environ["MHIP_GEMM_TILE"]
    assert c.shape == (M, N)
    rows = np.unique(np.r_[0, 127, 128, 255, 256, M - 1, rng.integers(0, M, 42)])
    A = as_f64(a).T if ta else as_f64(a)
    B = as_f64(b).T if tb else as_f64(b)
    exp = np.maximum(A[rows] @ B + as_f64(bias)[None, :], 0.0)
    assert_close(c[rows], exp, TOL[dtype], f"gemm {shape} {layout}")
    # the other kernel (128x128 tiles) accumulates each k-block in the same order
    os.environ["MHIP_GEMM_TILE"] = "128"
    try:
        c128 = kernels.matmul(a, b, bias, "relu", trans_a=ta, trans_b=tb)
    finally:
        del os.environ["MHIP_GEMM_TILE"]
    assert torch.equal(c, c128)


# Shapes with >= 192 tiles of 256x288 (as above for the ring of four).
NINE_BLOCKS = [(8192, 2304, 32), (7944, 2312, 96), (8192, 1736, 160), (6152, 2304, 448), (8192, 2304, 768),
               (8192, 2024, 1056), (8192, 2309, 192)]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=lambda d: NAME[d])
@pytest.mark.parametrize("layout", [(False, False), (False, True), (True, False), (True, True)],
                         ids=["nn", "nt", "tn", "tt"])
@pytest.mark.parametrize("shape", NINE_BLOCKS, ids=lambda s: "x".join(map(str, s)))
def test_gemm_256x288_tile(shape, layout, dtype, lib, monkeypatch):
    """The member whose four waves lie one above the other and all read the whole B tile (two of a
    wave's eighteen accumulator blocks in ordinary registers): bias, activation and residual, against
    the oracle on sampled rows and bit for bit against the 128x128 kernel; nothing is written behind
    the last row."""
    from metalhlo_amd import kernels
    M, N, K = shape
    ta, tb = layout
    if not ((not ta or M % 8 == 0) and (tb or N % 8 == 0)):
        pytest.skip("operand rows off 16-byte boundaries run the scalar kernel")
    a, b = _ab(M, N, K, dtype, 45, ta, tb)
    rng = np.random.default_rng(46)
    bias = to_dev(rng.standard_normal(N) * 0.5, dtype)
    r = to_dev(rng.standard_normal((M, N)), dtype)
    monkeypatch.setenv("MHIP_GEMM_TILE", "2570")
    guard = torch.full((M * N + 64,), 7.0, dtype=dtype, device="cuda")
    c = kernels.matmul(a, b, bias, "gelu", trans_a=ta, trans_b=tb, out=guard[:M * N].view(M, N))
    assert lib.mhip_gemm_last_variant() == 2570
    cr = kernels.matmul(a, b, bias, "none", trans_a=ta, trans_b=tb, residual=r)
    assert lib.mhip_gemm_last_variant() == 2570
    assert torch.all(guard[M * N:] == 7.0)
    monkeypatch.setenv("MHIP_GEMM_TILE", "128")
    assert torch.equal(c, kernels.matmul(a, b, bias, "gelu", trans_a=ta, trans_b=tb))
    assert torch.equal(cr, kernels.matmul(a, b, bias, "none", trans_a=ta, trans_b=tb, residual=r))
    rows = np.unique(np.r_[0, 31, 32, 63, 64, 255, 256, M - 1, rng.integers(0, M, 40)])
    A = as_f64(a).T if ta else as_f64(a)
    B = as_f64(b).T if tb else as_f64(b)
    exp = oracle.matmul_bias_act(A[rows], B, as_f64(bias), "gelu")
    assert_close(c[rows], exp, TOL[dtype], f"gemm 256x288 {shape} {layout}")
    exp = oracle.matmul_bias_act(A[rows], B, as_f64(bias), "none")
    exp = as_f64(to_dev(exp, dtype).cpu()) + as_f64(r)[rows]          # product rounded, then the residual added
    assert_close(cr[rows], exp, TOL[dtype], f"gemm 256x288 + residual {shape} {layout}")


# Shapes with >= 192 tiles of 128x192 (single stage, exits at every position of the unrolled ring of six,
# several trips; M and N ragged against the tile and, once, N odd).
SMALL_ROWS = [(8192, 768, 32), (4104, 1160, 96), (8192, 776, 160), (6152, 960, 224), (8192, 768, 768), (4096, 1544, 1056),
              (8192, 773, 192), (8192, 768, 3072)]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=lambda d: NAME[d])
@pytest.mark.parametrize("layout", [(False, False), (False, True), (True, False), (True, True)],
                         ids=["nn", "nt", "tn", "tt"])
@pytest.mark.parametrize("shape", SMALL_ROWS, ids=lambda s: "x".join(map(str, s)))
def test_gemm_128x192_tile(shape, layout, dtype, lib, monkeypatch):
    """The 128-row member of the family (B's 192 columns in a 256-column layout whose last quarter is
    never loaded): bias, activation and residual, against the oracle on sampled rows and bit for bit
    against the 128x128 kernel; nothing is written behind the last row."""
    from metalhlo_amd import kernels
    M, N, K = shape
    ta, tb = layout
    if not ((not ta or M % 8 == 0) and (tb or N % 8 == 0)):
        pytest.skip("operand rows off 16-byte boundaries run the scalar kernel")
    a, b = _ab(M, N, K, dtype, 43, ta, tb)
    rng = np.random.default_rng(44)
    bias = to_dev(rng.standard_normal(N) * 0.5, dtype)
    r = to_dev(rng.standard_normal((M, N)), dtype)
    monkeypatch.setenv("MHIP_GEMM_TILE", "2569")
    guard = torch.full((M * N + 64,), 7.0, dtype=dtype, device="cuda")
    c = kernels.matmul(a, b, bias, "silu", trans_a=ta, trans_b=tb, out=guard[:M * N].view(M, N))
    assert lib.mhip_gemm_last_variant() == 2569
    cr = kernels.matmul(a, b, bias, "none", trans_a=ta, trans_b=tb, residual=r)
    assert lib.mhip_gemm_last_variant() == 2569
    assert torch.all(guard[M * N:] == 7.0)
    monkeypatch.setenv("MHIP_GEMM_TILE", "128")
    assert torch.equal(c, kernels.matmul(a, b, bias, "silu", trans_a=ta, trans_b=tb))
    assert torch.equal(cr, kernels.matmul(a, b, bias, "none", trans_a=ta, trans_b=tb, residual=r))
    rows = np.unique(np.r_[0, 31, 32, 63, 64, 127, 128, M - 1, rng.integers(0, M, 40)])
    A = as_f64(a).T if ta else as_f64(a)
    B = as_f64(b).T if tb else as_f64(b)
    exp = oracle.matmul_bias_act(A[rows], B, as_f64(bias), "silu")
    assert_close(c[rows], exp, TOL[dtype], f"gemm 128x192 {shape} {layout}")
    exp = oracle.matmul_bias_act(A[rows], B, as_f64(bias), "none")
    exp = as_f64(to_dev(exp, dtype).cpu()) + as_f64(r)[rows]          # product rounded, then the residual added
    assert_close(cr[rows], exp, TOL[dtype], f"gemm 128x192 + residual {shape} {layout}")


@pytest.mark.parametrize("tile", ["2560", "2561", "2567", "2568", "2569", "2570"],
                         ids=["256x256", "256x128", "256x384", "256x128-two-per-cu", "128x192", "256x288"])
def test_gemm_ring_kernels_batched(tile, lib, monkeypatch):
    """The ring kernels on a strided batch (one grid row per matrix): every batch element against the
    oracle on sampled rows and bit for bit against the 128x128 kernel."""
    from metalhlo_amd import kernels
    M, N, K, B = 2048, 2312, 224, 4            # 8 x 7 x 4 = 224 tiles of 256x384, ragged in N
    a, b = _ab(M, N, K, torch.bfloat16, 51, batch=(B,))
    rng = np.random.default_rng(52)
    bias = to_dev(rng.standard_normal(N) * 0.5, torch.bfloat16)
    monkeypatch.setenv("MHIP_GEMM_TILE", tile)
    c = kernels.matmul(a, b, bias, "relu")
    assert lib.mhip_gemm_last_variant() == int(tile)
    monkeypatch.setenv("MHIP_GEMM_TILE", "128")
    assert torch.equal(c, kernels.matmul(a, b, bias, "relu"))
    rows = np.r_[0, 255, 256, M - 1, rng.integers(0, M, 12)]
    for i in range(B):
        exp = oracle.matmul_bias_act(as_f64(a[i])[rows], as_f64(b[i]), as_f64(bias), "relu")
        assert_close(c[i][rows], exp, 2e-2, f"batched {tile} element {i}")


# Shapes with >= 192 tiles of 256x384 (K stages of 32: a single stage, exits at every position of the
# unrolled ring of four, several trips; M and N ragged against the tile and, once, N odd).
WIDEST = [(8192, 2304, 32), (7944, 2408, 96), (8192, 2696, 160), (7680, 3072, 448), (8192, 2304, 768),
          (6152, 3080, 1056), (8192, 2309, 192)]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=lambda d: NAME[d])
@pytest.mark.parametrize("layout", [(False, False), (False, True), (True, False), (True, True)],
                         ids=["nn", "nt", "tn", "tt"])
@pytest.mark.parametrize("shape", WIDEST, ids=lambda s: "x".join(map(str, s)))
def test_gemm_256x384_tile(shape, layout, dtype, lib, monkeypatch):
    """The widest member of the family (eight of a wave's 24 accumulator blocks live in ordinary
    registers, B is held as a 256-column and a 128-column tile): bias, activation and residual,
    against the oracle on sampled rows and bit for bit against the 128x128 kernel, which
    accumulates every k-block in the same order; nothing is written behind the last row."""
    from metalhlo_amd import kernels
    M, N, K = shape
    ta, tb = layout
    aligned = (not ta or M % 8 == 0) and (tb or N % 8 == 0)
    if not aligned:
        pytest.skip("operand rows off 16-byte boundaries run the scalar kernel")
    a, b = _ab(M, N, K, dtype, 41, ta, tb)
    rng = np.random.default_rng(42)
    bias = to_dev(rng.standard_normal(N) * 0.5, dtype)
    r = to_dev(rng.standard_normal((M, N)), dtype)
    monkeypatch.setenv("MHIP_GEMM_TILE", "2567")
    guard = torch.full((M * N + 64,), 7.0, dtype=dtype, device="cuda")
    c = kernels.matmul(a, b, bias, "gelu", trans_a=ta, trans_b=tb, out=guard[:M * N].view(M, N))
    assert lib.mhip_gemm_last_variant() == 2567
    cr = kernels.matmul(a, b, bias, "relu", trans_a=ta, trans_b=tb, residual=r)
    assert lib.mhip_gemm_last_variant() == 2567
    assert torch.all(guard[M * N:] == 7.0)
    monkeypatch.setenv("MHIP_GEMM_TILE", "128")
    assert torch.equal(c, kernels.matmul(a, b, bias, "gelu", trans_a=ta, trans_b=tb))
    assert torch.equal(cr, kernels.matmul(a, b, bias, "relu", trans_a=ta, trans_b=tb, residual=r))
    rows = np.unique(np.r_[0, 31, 32, 127, 128, 255, 256, M - 1, rng.integers(0, M, 40)])
    A = as_f64(a).T if ta else as_f64(a)
    B = as_f64(b).T if tb else as_f64(b)
    exp = oracle.matmul_bias_act(A[rows], B, as_f64(bias), "gelu")
    assert_close(c[rows], exp, TOL[dtype], f"gemm 256x384 {shape} {layout}")
    exp = oracle.matmul_bias_act(A[rows], B, as_f64(bias), "relu")
    exp = as_f64(to_dev(exp, dtype).cpu()) + as_f64(r)[rows]          # product rounded, then the residual added
    assert_close(cr[rows], exp, TOL[dtype], f"gemm 256x384 + residual {shape} {layout}")
    # an activation its epilogue does not serve goes to another kernel
    monkeypatch.setenv("MHIP_GEMM_TILE", "2567")
    kernels.matmul(a, b, bias, "silu", trans_a=ta, trans_b=tb)
    assert lib.mhip_gemm_last_variant() != 2567


@pytest.mark.parametrize("tile", ["2560", "2561"], ids=["256x256", "256x128"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=lambda d: NAME[d])
def test_gemm_ring_kernel_rows_of_c_at_any_alignment(tile, dtype, monkeypatch):
    """N that is no multiple of 8 (odd, and even but not a multiple of 4) with B stored [N, K]: the
    rows of C start at arbitrary even bytes and end in a partial chunk.  Bias, activation and
    residual included; compared with the 128x128 kernel (2-byte stores there) bit for bit and
    with the oracle on sampled rows; nothing is written behind the last row."""
    from metalhlo_amd import kernels
    rng = np.random.default_rng(33)
    for (M, N, K, ta) in [(4000, 3081, 512, False), (3904, 3203, 544, True), (4096, 3090, 512, False)]:
        a, b = _ab(M, N, K, dtype, 34, ta, True)
        bias = to_dev(rng.standard_normal(N) * 0.5, dtype)
        r = to_dev(rng.standard_normal((M, N)), dtype)
        monkeypatch.setenv("MHIP_GEMM_TILE", tile)
        c = kernels.matmul(a, b, bias, "gelu", trans_a=ta, trans_b=True, residual=r)
        guard = torch.full((M * N + 64,), 7.0, dtype=dtype, device="cuda")
        kernels.matmul(a, b, bias, "gelu", trans_a=ta, trans_b=True, out=guard[:M * N].view(M, N))
        assert torch.all(guard[M * N:] == 7.0)
        monkeypatch.setenv("MHIP_GEMM_TILE", "128")
        c128 = kernels.matmul(a, b, bias, "gelu", trans_a=ta, trans_b=True, residual=r)
        assert torch.equal(c, c128), (M, N, K, ta)
        rows = np.unique(np.r_[0, 1, 255, 256, M - 1, rng.integers(0, M, 20)])
        A = as_f64(a).T if ta else as_f64(a)
        exp = oracle.matmul_bias_act(A[rows], as_f64(b).T, as_f64(bias), "gelu")
        assert_close(guard[:M * N].view(M, N)[rows], exp, TOL[dtype], f"odd N {(M, N, K)}")
        exp = as_f64(to_dev(exp, dtype).cpu()) + as_f64(r)[rows]                     # product rounded, then the residual added
        assert_close(c[rows], exp, TOL[dtype], f"odd N + residual {(M, N, K)}")


# More 256x128 tiles than compute units, M a multiple of 256, N of 128, K >= 640: the persistent
# workgroups that store a tile inside the loop of the next one (several tiles per workgroup, a
# last round that is not full, K that leaves the straight-line part at once or after some trips).
STREAMED = [(8192, 3072, 768), (2304, 4096, 640), (4096, 8320, 1024), (8192, 2304, 2080)]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=lambda d: NAME[d])
@pytest.mark.parametrize("tb", [False, True], ids=["nn", "nt"])
@pytest.mark.parametrize("shape", STREAMED, ids=lambda s: "x".join(map(str, s)))
def test_gemm_streamed_tiles(shape, tb, dtype, monkeypatch):
    """Forced, and compared with the oracle on sampled rows of every tile row and bit for bit with
    the plain 256x128 kernel; with and without bias, GELU epilogue; nothing written outside C."""
    from metalhlo_amd import kernels
    M, N, K = shape
    a, b = _ab(M, N, K, dtype, 61, False, tb)
    rng = np.random.default_rng(62)
    bias = to_dev(rng.standard_normal(N) * 0.5, dtype)
    for use_bias, act in ((True, "gelu"), (False, "none")):
        bb = bias if use_bias else None
        monkeypatch.setenv("MHIP_GEMM_TILE", "2562")
        guard = torch.full((M * N + 4096,), 7.0, dtype=dtype, device="cuda")
        c = kernels.matmul(a, b, bb, act, trans_b=tb, out=guard[2048:2048 + M * N].view(M, N))
        assert torch.all(guard[:2048] == 7.0) and torch.all(guard[2048 + M * N:] == 7.0)
        monkeypatch.setenv("MHIP_GEMM_TILE", "2561")
        plain = kernels.matmul(a, b, bb, act, trans_b=tb)
        assert torch.equal(c, plain), (shape, tb, use_bias)
        rows = np.unique(np.r_[np.arange(0, M, 256), np.arange(255, M, 256), rng.integers(0, M, 24)])
        B = as_f64(b).T if tb else as_f64(b)
        exp = oracle.matmul_bias_act(as_f64(a)[rows], B, as_f64(bias) if use_bias else None, act)
        assert_close(c[rows], exp, TOL[dtype], f"streamed gemm {shape} nt={tb} bias={use_bias}")


def test_gemm_streamed_tiles_agree_with_the_default_choice(lib):
    """[8192, 768] x [768, 3584] (three and a half rounds of narrow tiles, no column split with a
    band of at most one round): the default choice (wide tiles) and the streamed kernel give the
    same bits, and a problem the streamed kernel cannot take (ragged N) still runs when it is forced."""
    from metalhlo_amd import kernels
    a, b = _ab(8192, 3584, 768, torch.bfloat16, 63)
    os.environ.pop("MHIP_GEMM_TILE", None)
    c = kernels.matmul(a, b, None, "gelu")
    os.environ["MHIP_GEMM_TILE"] = "2562"
    try:
        forced = kernels.matmul(a, b, None, "gelu")
        a2, b2 = _ab(8192, 3000, 768, torch.bfloat16, 64)
        ragged = kernels.matmul(a2, b2)
    finally:
        del os.environ["MHIP_GEMM_TILE"]
    assert torch.equal(c, forced)
    assert torch.equal(ragged, kernels.matmul(a2, b2))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=lambda d: NAME[d])
@pytest.mark.parametrize("tb", [False, True], ids=["nn", "nt"])
@pytest.mark.parametrize("shape", [(8192, 2304, 768), (4096, 4360, 512), (2048, 8200, 96)], ids=lambda s: "x".join(map(str, s)))
def test_gemm_wide_tiles_plus_a_narrow_band(shape, tb, dtype, monkeypatch):
    """Forced: wide tiles on the columns that make whole rounds, 256x128 tiles on the rest (the
    band ragged in two of the shapes).  Bit for bit the wide kernel's result, with bias + GELU and
    with a residual; nothing written outside C; sampled rows against the oracle."""
    from metalhlo_amd import kernels
    M, N, K = shape
    a, b = _ab(M, N, K, dtype, 65, False, tb)
    rng = np.random.default_rng(66)
    bias = to_dev(rng.standard_normal(N) * 0.5, dtype)
    res = to_dev(rng.standard_normal((M, N)), dtype)
    for use_bias, act, r in ((True, "gelu", None), (False, "none", res)):
        bb = bias if use_bias else None
        monkeypatch.setenv("MHIP_GEMM_TILE", "2563")
        guard = torch.full((M * N + 4096,), 7.0, dtype=dtype, device="cuda")
        c = kernels.matmul(a, b, bb, act, trans_b=tb, residual=r, out=guard[2048:2048 + M * N].view(M, N))
        assert torch.all(guard[:2048] == 7.0) and torch.all(guard[2048 + M * N:] == 7.0)
        monkeypatch.setenv("MHIP_GEMM_TILE", "2560")
        wide = kernels.matmul(a, b, bb, act, trans_b=tb, residual=r)
        assert torch.equal(c, wide), (shape, tb, use_bias)
        if r is None:
            rows = np.unique(np.r_[np.arange(0, M, 256), np.arange(255, M, 256), rng.integers(0, M, 24)])
            B = as_f64(b).T if tb else as_f64(b)
            exp = oracle.matmul_bias_act(as_f64(a)[rows], B, as_f64(bias) if use_bias else None, act)
            assert_close(c[rows], exp, TOL[dtype], f"split gemm {shape} nt={tb}")


def test_gemm_one_round_of_the_widest_tile_is_the_default_where_it_saves_a_round(lib, monkeypatch):
    """[8192, 768] x [768, 2304] and x [768, 3072]: 192 and 256 tiles of 256x384 (one round) against
    two rounds of wide or three of narrow tiles -- the default with an activation the widest tile's
    epilogue serves; with another one (silu) the column split as before; [8192, 768] x [768, 12288]
    (four rounds against six) stays on wide tiles.  Always the bits of the forced choice."""
    from metalhlo_amd import kernels
    kernels.tuning_clear()                 # the heuristic's choice, not a table entry's
    for N in (2304, 3072):
        a, b = _ab(8192, N, 768, torch.bfloat16, 67)
        for act, variant in (("gelu", 2567), ("none", 2567), ("silu", 2563)):
            monkeypatch.delenv("MHIP_GEMM_TILE", raising=False)
            c = kernels.matmul(a, b, None, act)
            assert lib.mhip_gemm_last_variant() == variant, (N, act)
            monkeypatch.setenv("MHIP_GEMM_TILE", str(variant))
            assert torch.equal(c, kernels.matmul(a, b, None, act))
    a, b = _ab(8192, 12288, 768, torch.bfloat16, 68)
    monkeypatch.delenv("MHIP_GEMM_TILE", raising=False)
    kernels.matmul(a, b)
    assert lib.mhip_gemm_last_variant() == 2560
    # 768 columns: 192 tiles of 256x128 would leave a quarter of the device idle, 256 of 128x192 do not
    for K in (768, 3072):
        a, b = _ab(8192, 768, K, torch.bfloat16, 69)
        monkeypatch.delenv("MHIP_GEMM_TILE", raising=False)
        c = kernels.matmul(a, b)
        assert lib.mhip_gemm_last_variant() == 2569, K
        monkeypatch.setenv("MHIP_GEMM_TILE", "2561")
        assert torch.equal(c, kernels.matmul(a, b))


def test_gemm_streaming_stores_of_a_large_result(monkeypatch):
    """A result of more than 256 MB is stored with the streaming hint; forced here on small
    problems (both tile widths, aligned and odd N, with a residual): the same bits, nothing
    written outside C."""
    from metalhlo_amd import kernels
    rng = np.random.default_rng(68)
    for (M, N, K, tile, tb) in [(4096, 4096, 256, "2560", False), (8192, 768, 512, "2561", False), (2048, 6145, 128, "2560", True)]:
        a, b = _ab(M, N, K, torch.bfloat16, 69, False, tb)
        bias = to_dev(rng.standard_normal(N) * 0.5, torch.bfloat16)
        res = to_dev(rng.standard_normal((M, N)), torch.bfloat16)
        monkeypatch.setenv("MHIP_GEMM_TILE", tile)
        for r in (None, res):
            monkeypatch.setenv("MHIP_GEMM_STREAM_C", "2")
            plain = kernels.matmul(a, b, bias, "gelu", trans_b=tb, residual=r)
            monkeypatch.setenv("MHIP_GEMM_STREAM_C", "3")
            guard = torch.full((M * N + 4096,), 7.0, dtype=torch.bfloat16, device="cuda")
            c = kernels.matmul(a, b, bias, "gelu", trans_b=tb, residual=r, out=guard[2048:2048 + M * N].view(M, N))
            assert torch.all(guard[:2048] == 7.0) and torch.all(guard[2048 + M * N:] == 7.0)
            assert torch.equal(c, plain), (M, N, K, tile)


def test_gemm_large_exact_small_integers():
    """Integer-valued operands with exactly representable partial sums: bit-exact."""
    from metalhlo_amd import kernels
    rng = np.random.default_rng(29)
    a = to_dev(rng.integers(-3, 4, (4096, 512)).astype(np.float64), torch.bfloat16)
    b = to_dev(rng.integers(-3, 4, (512, 4096)).astype(np.float64), torch.bfloat16)
    c = kernels.matmul(a, b)
    exp = (a.double() @ b.double())
    assert torch.equal(c.double(), exp.to(torch.bfloat16).double())
    assert torch.equal(kernels.matmul(a, b.t().contiguous(), trans_b=True), c)


@pytest.mark.parametrize("tile", ["128", "256", "2560", "2561", "simple"])
def test_gemm_residual_equals_gemm_then_add(tile, monkeypatch):
    """act(A.B + bias) + R in one kernel is bit for bit mhip_gemm followed by mhip_add, on every
    GEMM kernel (tile choice forced), batched and in place (R == C)."""
    from metalhlo_amd import kernels
    rng = np.random.default_rng(48)
    for (batch, M, N, K, act) in [(1, 512, 768, 320, "none"), (3, 300, 264, 96, "gelu"), (1, 8192, 768, 768, "none")]:
        if tile == "simple":
            N += 1                                   # odd N: 16-byte paths off
        else:
            monkeypatch.setenv("MHIP_GEMM_TILE", tile)
        shape_a, shape_b = ((batch, M, K), (batch, K, N)) if batch > 1 else ((M, K), (K, N))
        a = to_dev(rng.standard_normal(shape_a), torch.bfloat16)
        b = to_dev(rng.standard_normal(shape_b) * 0.1, torch.bfloat16)
        bias = to_dev(rng.standard_normal(N), torch.bfloat16)
        r = to_dev(rng.standard_normal(shape_a[:-1] + (N,)), torch.bfloat16)
        two = kernels.add(kernels.matmul(a, b, bias=bias, activation=act), r)
        one = kernels.matmul(a, b, bias=bias, activation=act, residual=r)
        assert torch.equal(one, two), f"{tile} {(batch, M, N, K, act)}"
        inplace = r.clone()
        kernels.matmul(a, b, bias=bias, activation=act, residual=inplace, out=inplace)
        assert torch.equal(inplace, two), f"in place, {tile} {(batch, M, N, K, act)}"
    f = to_dev(rng.standard_normal((33, 17)), torch.float32)
    g = to_dev(rng.standard_normal((17, 9)), torch.float32)
    r = to_dev(rng.standard_normal((33, 9)), torch.float32)
    assert torch.equal(kernels.matmul(f, g, residual=r), kernels.add(kernels.matmul(f, g), r))


@pytest.mark.parametrize("dtype", [torch.int32, torch.int64, torch.float64], ids=["i32", "i64", "f64"])
def test_gemm_exact_types(dtype):
    """i32 / i64 products wrap around like the CPU's; f64 accumulates in f64 (checked to 1e-12)."""
    from metalhlo_amd import kernels
    rng = np.random.default_rng(31)
    for (batch, M, N, K, ta, tb) in [((), 33, 17, 45, False, False), ((3,), 20, 31, 16, True, False), ((2,), 7, 5, 130, False, True)]:
        sa = batch + ((K, M) if ta else (M, K))
        sb = batch + ((N, K) if tb else (K, N))
        if dtype == torch.float64:
            a, b = torch.from_numpy(rng.standard_normal(sa)), torch.from_numpy(rng.standard_normal(sb))
        else:
            hi = 2 ** 20 if dtype == torch.int32 else 2 ** 40                    # products overflow: wrap-around is exercised
            a = torch.from_numpy(rng.integers(-hi, hi, sa)).to(dtype)
            b = torch.from_numpy(rng.integers(-hi, hi, sb)).to(dtype)
        ea = a.transpose(-1, -2) if ta else a
        eb = b.transpose(-1, -2) if tb else b
        if dtype == torch.float64:
            e = ea @ eb
        else:                                                                    # numpy integer matmul wraps
            e = torch.from_numpy(np.matmul(ea.numpy(), eb.numpy()))
        got = kernels.matmul(a.cuda(), b.cuda(), trans_a=ta, trans_b=tb).cpu()
        if dtype == torch.float64:
            assert torch.allclose(got, e, rtol=1e-12, atol=1e-12)
        else:
            assert torch.equal(got, e)


def test_gemm_errors(lib):
    assert lib.mhip_gemm(None, None, None, None, None, 4, 4, 4, 1, 0, 0, 0, 0, 0, 0, 3) == 1
    x = torch.zeros(4, 4, dtype=torch.int32, device="cuda")
    p = x.data_ptr()
    assert lib.mhip_gemm(None, p, p, None, p, 4, 4, 4, 1, 0, 0, 0, 0, 0, 0, 5) == 2   # int8 unsupported
    assert lib.mhip_gemm(None, p, p, None, p, 4, 4, 4, 1, 0, 0, 0, 0, 0, 1, 7) == 2   # no activation on int32
    assert lib.mhip_gemm(None, p, p, None, p, 4, 4, 4, 1, 0, 0, 0, 0, 0, 99, 1) == 1  # bad activation
    assert lib.mhip_gemm(None, p, p, None, p, 0, 4, 4, 1, 0, 0, 0, 0, 0, 0, 1) == 0   # empty is a no-op


def test_gemm_ring_kernel_takes_wide_and_deep_operands(lib):
    """The ring kernels address their operands with 32-bit byte offsets, so eligibility is decided
    by the operands' real extents: B stored [K, N] with N = 50304 (an untied vocabulary head,
    77 MB) and [2048, 32768] x [32768, 8192] stay on the four-wave ring kernel (variant 2560 / 2561), and the
    results follow the oracle on sampled rows."""
    from metalhlo_amd import kernels
    rng = np.random.default_rng(71)
    for (M, N, K) in [(4096, 50304, 768), (2048, 8192, 32768)]:
        a = to_dev(rng.uniform(-1, 1, (M, K)), torch.bfloat16)
        b = to_dev(rng.uniform(-1, 1, (K, N)) * (K ** -0.5), torch.bfloat16)
        c = kernels.matmul(a, b)
        assert 2560 <= lib.mhip_gemm_last_variant() <= 2570, (M, N, K, lib.mhip_gemm_last_variant())
        rows = np.r_[0, 255, 256, M - 1, rng.integers(0, M, 12)]
        assert_close(c[rows], as_f64(a[rows]) @ as_f64(b), 2e-2, f"gemm {M}x{N}x{K}")
    # fp32 operands run none of the 16-bit variants
    kernels.matmul(torch.ones(64, 64, device="cuda"), torch.ones(64, 64, device="cuda"))
    assert lib.mhip_gemm_last_variant() == 0
