"""GPU parity: flash-attention forward through the C-ABI vs the float64
materialised-scores oracle.  fp32: 1e-5 relative; bf16/fp16: 2e-2 relative
(floor max(tol, tol*|e|))."""
import math

import ctypes as C

import numpy as np
import pytest
import torch

from oracle import oracle
from tests.util import NAME, TOL, as_f64, assert_close, to_dev

pytestmark = pytest.mark.gpu


def _qkv(B, H, Sq, Skv, D, dtype, seed):
    rng = np.random.default_rng(seed)
    q = to_dev(rng.standard_normal((B, H, Sq, D)), dtype)
    k = to_dev(rng.standard_normal((B, H, Skv, D)), dtype)
    v = to_dev(rng.standard_normal((B, H, Skv, D)), dtype)
    return q, k, v


def test_c1_fp32_causal_sdpa():
    """The first benchmark configuration: fp32, B1 H4 S128 D64, causal, scale 1/8, seed 1234 —
    causal flag and additive -inf mask variants must both match the oracle."""
    from metalhlo_amd import kernels
    q, k, v = _qkv(1, 4, 128, 128, 64, torch.float32, 1234)
    exp = oracle.attention(as_f64(q), as_f64(k), as_f64(v), scale=0.125, is_causal=True)
    o = kernels.flash_attention(q, k, v, scale=0.125, is_causal=True)
    assert o.shape == (1, 4, 128, 64)
    assert_close(o, exp, 1e-5, "C1 causal flag")
    m = np.where(np.arange(128)[None, :] > np.arange(128)[:, None], -np.inf, 0.0)
    om = kernels.flash_attention(q, k, v, scale=0.125, mask=to_dev(m, torch.float32))
    assert_close(om, exp, 1e-5, "C1 additive mask")
    # causal row 0 attends to key 0 only
    assert_close(o[:, :, 0], as_f64(v)[:, :, 0], 1e-6, "row 0 == V[0]")


F32_CASES = [  # B, H, Sq, Skv, D, causal -- the fp32 matrix-instruction kernel (head sizes 32 .. 128)
    (1, 4, 128, 128, 64, True), (2, 2, 256, 256, 128, False), (1, 3, 200, 333, 96, False),
    (1, 2, 77, 333, 64, True), (1, 2, 333, 77, 32, True), (1, 1, 1, 1, 128, True), (2, 2, 130, 31, 64, False),
    (1, 2, 1024, 1024, 64, True),
]


@pytest.mark.parametrize("case", F32_CASES, ids=lambda c: "B%dH%dq%dk%dD%d%s" % (*c[:5], "c" if c[5] else ""))
def test_attention_f32_matrix_cores(case, monkeypatch):
    """fp32 tensors on v_mfma_f32_32x32x2_f32: 1e-5 against the oracle (ragged query and key counts,
    causal with more queries than keys and the other way round), and the scalar kernel it
    replaces stays within the same bar of it."""
    from metalhlo_amd import kernels
    B, H, Sq, Skv, D, causal = case
    q, k, v = _qkv(B, H, Sq, Skv, D, torch.float32, 71)
    exp = oracle.attention(as_f64(q), as_f64(k), as_f64(v), is_causal=causal)
    o = kernels.flash_attention(q, k, v, is_causal=causal)
    assert_close(o, exp, 1e-5, f"fp32 attention {case}")
    monkeypatch.setenv("MHIP_FA_F32_MFMA", "2")
    scalar = kernels.flash_attention(q, k, v, is_causal=causal)
    assert_close(scalar, exp, 1e-5, f"fp32 scalar attention {case}")
    assert not torch.equal(o, scalar) or Sq * Skv <= 1        # two kernels, two summation orders


def test_attention_f32_matrix_cores_mask_and_scale():
    from metalhlo_amd import kernels
    rng = np.random.default_rng(72)
    q, k, v = _qkv(2, 3, 160, 200, 64, torch.float32, 73)
    for shape in [(2, 3, 160, 200), (2, 1, 160, 200), (1, 1, 160, 200)]:
        m = rng.standard_normal(shape)
        m[..., :, 150:] = -np.inf
        md = to_dev(m, torch.float32)
        o = kernels.flash_attention(q, k, v, mask=md, scale=0.07)
        exp = oracle.attention(as_f64(q), as_f64(k), as_f64(v), scale=0.07, mask=as_f64(md))
        assert_close(o, exp, 1e-5, f"fp32 mask {shape}")
    m = np.zeros((1, 1, 160, 200)); m[..., 7, :] = -np.inf
    md = to_dev(m, torch.float32)
    o = kernels.flash_attention(q, k, v, mask=md, is_causal=True, scale=-0.1)
    exp = oracle.attention(as_f64(q), as_f64(k), as_f64(v), scale=-0.1, is_causal=True, mask=as_f64(md))
    assert_close(o, exp, 1e-5, "fp32 mask + causal, negative scale")
    assert torch.count_nonzero(o[:, :, 7]) == 0                # a fully masked row gives zeros
    # large logits: the running maximum keeps the exponentials in range (the fp32 rounding of a
    # logit of size L alone is worth about L * 1e-6 relative in its probability, so 1e-5 holds
    # for logits of the usual size only; at 30 x 30 the result must still be finite and close)
    big = kernels.flash_attention(q * 3, k * 3, v)
    assert_close(big, oracle.attention(as_f64(q) * 3, as_f64(k) * 3, as_f64(v)), 1e-4, "fp32 larger logits")
    huge = kernels.flash_attention(q * 30, k * 30, v)
    assert torch.isfinite(huge).all()
    assert_close(huge, oracle.attention(as_f64(q) * 30, as_f64(k) * 30, as_f64(v)), 2e-3, "fp32 huge logits")


CASES = [  # B, H, Sq, Skv, D, causal
    (1, 2, 128, 128, 128, False), (1, 2, 128, 128, 128, True),
    (2, 3, 256, 256, 64, True), (2, 3, 256, 256, 64, False),
    (1, 8, 200, 200, 128, True),      # ragged: S not a multiple of the 128/64 tiles
    (1, 2, 77, 333, 64, False),       # cross attention, ragged both ways
    (1, 1, 333, 77, 128, True),       # more queries than keys (rows past Skv see every key)
    (1, 8, 1024, 1024, 64, True),     # GPT-2-small head shape
    (2, 2, 96, 160, 32, True),        # head size without an MFMA path
    (1, 1, 1, 1, 128, True),
]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=lambda d: NAME[d])
@pytest.mark.parametrize("case", CASES, ids=lambda c: "B%dH%dq%dk%dD%d%s" % (*c[:5], "c" if c[5] else ""))
def test_attention_16bit(case, dtype):
    from metalhlo_amd import kernels
    B, H, Sq, Skv, D, causal = case
    q, k, v = _qkv(B, H, Sq, Skv, D, dtype, 41)
    o = kernels.flash_attention(q, k, v, is_causal=causal)
    exp = oracle.attention(as_f64(q), as_f64(k), as_f64(v), is_causal=causal)
    assert_close(o, exp, TOL[dtype], f"attention {case}")


def test_attention_mask_scale_variants():
    from metalhlo_amd import kernels
    rng = np.random.default_rng(42)
    q, k, v = _qkv(2, 4, 192, 192, 128, torch.bfloat16, 43)
    # per-(b,h) mask, broadcast-over-heads mask, broadcast-over-everything mask
    for shape in [(2, 4, 192, 192), (2, 1, 192, 192), (1, 1, 192, 192)]:
        m = rng.standard_normal(shape)
        m[..., :, 100:] = -np.inf          # padded keys
        md = to_dev(m, torch.bfloat16)
        o = kernels.flash_attention(q, k, v, mask=md, scale=0.05)
        exp = oracle.attention(as_f64(q), as_f64(k), as_f64(v), scale=0.05, mask=as_f64(md))
        assert_close(o, exp, 2e-2, f"mask {shape}")
    # mask + causal together, negative scale, fully masked rows -> zeros
    m = np.zeros((1, 1, 192, 192)); m[..., 5, :] = -np.inf
    md = to_dev(m, torch.bfloat16)
    o = kernels.flash_attention(q, k, v, mask=md, is_causal=True, scale=-0.1)
    exp = oracle.attention(as_f64(q), as_f64(k), as_f64(v), scale=-0.1, is_causal=True, mask=as_f64(md))
    assert_close(o, exp, 2e-2, "mask+causal, negative scale")
    assert torch.count_nonzero(o[:, :, 5]) == 0


PIPE_CASES = [  # B, H, Sq, Skv, causal -- head size 128, bf16, at least 256 query rows
    (1, 2, 256, 64, False),       # a single key block
    (1, 2, 512, 1000, False),     # last key block partly filled
    (2, 3, 777, 777, True),       # ragged causal, even number of query tiles
    (1, 2, 1280, 1280, True),     # odd number of query tiles: the middle one is not paired
    (1, 1, 300, 5, True),         # fewer keys than one block
    (1, 2, 640, 2048, True),      # causal with more keys than queries
    (1, 1, 333, 77, True),        # more queries than keys
    (1, 8, 2048, 2048, True),
]


@pytest.fixture
def force_pipelined(monkeypatch):
    """The 256-row pipelined kernel is normally chosen only for grids that fill the chip."""
    monkeypatch.setenv("MHIP_FA_PIPE", "3")
    return monkeypatch


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=lambda d: NAME[d])
@pytest.mark.parametrize("pair", [0, 1], ids=["one-tile", "paired-tiles"])
@pytest.mark.parametrize("case", PIPE_CASES, ids=lambda c: "B%dH%dq%dk%d%s" % (*c[:4], "c" if c[4] else ""))
def test_attention_pipelined_kernel(case, pair, dtype, force_pipelined):
    from metalhlo_amd import kernels
    B, H, Sq, Skv, causal = case
    if pair and not causal:
        pytest.skip("only causal workgroups pair tiles")
    force_pipelined.setenv("MHIP_FA_PAIR", str(pair))
    q, k, v = _qkv(B, H, Sq, Skv, 128, dtype, 46)
    o = kernels.flash_attention(q, k, v, is_causal=causal)
    exp = oracle.attention(as_f64(q), as_f64(k), as_f64(v), is_causal=causal)
    assert_close(o, exp, TOL[dtype], f"pipelined attention {case}")


def test_attention_pipelined_scale_and_extremes(force_pipelined):
    """Negative scale and widely spread scores on the 256-row kernel (bf16, head size 128)."""
    from metalhlo_amd import kernels
    q, k, v = _qkv(1, 2, 512, 512, 128, torch.bfloat16, 45)
    for causal in (False, True):
        o = kernels.flash_attention(q, k, v, is_causal=causal, scale=-0.07)
        exp = oracle.attention(as_f64(q), as_f64(k), as_f64(v), scale=-0.07, is_causal=causal)
        assert_close(o, exp, 2e-2, f"negative scale causal={causal}")
    # row maxima that keep growing along the keys (every block moves the running maximum)
    kk = k * torch.linspace(0.2, 6.0, 512, device="cuda").view(1, 1, 512, 1).to(torch.bfloat16)
    o = kernels.flash_attention(q, kk, v, scale=0.5)
    exp = oracle.attention(as_f64(q), as_f64(kk), as_f64(v), scale=0.5)
    assert_close(o, exp, 2e-2, "growing maxima")
    # the pipelined kernel and the 128-row kernel agree (same inputs, kernel choice forced)
    a = kernels.flash_attention(q, k, v, is_causal=True)
    force_pipelined.setenv("MHIP_FA_PIPE", "2")
    b = kernels.flash_attention(q, k, v, is_causal=True)
    assert_close(a, as_f64(b), 2e-2, "pipelined == 128-row kernel")
    # (both keep the same lazily moving reference maximum, so they usually agree to the last bit;
    # their row sums are taken in different orders, so that is not required)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=lambda d: NAME[d])
@pytest.mark.parametrize("D", [64, 128])
def test_attention_strided_views(D, dtype, lib):
    """Q, K, V read in place from a fused projection [B,S,3,H,D] and O written as [B,S,H,D]:
    the same numbers as packed tensors give, and the oracle's."""
    from metalhlo_amd import kernels
    B, H, S = 2, 3, 200
    rng = np.random.default_rng(47)
    qkv = to_dev(rng.standard_normal((B, S, 3, H, D)), dtype)
    q, k, v = qkv.permute(2, 0, 3, 1, 4).unbind(0)                 # [B,H,S,D] views, row pitch 3*H*D
    assert not q.is_contiguous()
    out = torch.full((B, S, H, D), float("nan"), dtype=dtype, device="cuda")
    for causal in (True, False):
        kernels.flash_attention(q, k, v, is_causal=causal, out=out.permute(0, 2, 1, 3))
        packed = kernels.flash_attention(q.contiguous(), k.contiguous(), v.contiguous(), is_causal=causal)
        assert torch.equal(out.permute(0, 2, 1, 3), packed), "strided and packed results differ"
        exp = oracle.attention(as_f64(q), as_f64(k), as_f64(v), is_causal=causal)
        assert_close(out.permute(0, 2, 1, 3), exp, TOL[dtype], f"strided attention D={D} causal={causal}")
    # layouts the strided entry refuses: fp32, odd strides
    x = torch.zeros(4096, dtype=torch.float32, device="cuda")
    p = x.data_ptr()
    st = (C.c_int64 * 12)(*([2048, 1024, 128] * 4))
    assert lib.mhip_flash_attention_strided(None, p, p, p, None, p, 1, 1, 8, 8, 64, 1.0, 0, 0, 0, 1, C.addressof(st)) == 2
    st = (C.c_int64 * 12)(*([2048, 1024, 100] * 4))
    assert lib.mhip_flash_attention_strided(None, p, p, p, None, p, 1, 1, 8, 8, 64, 1.0, 0, 0, 0, 3, C.addressof(st)) == 2
    st = (C.c_int64 * 12)(*([2048, 1024, 32] * 4))                 # rows would overlap
    assert lib.mhip_flash_attention_strided(None, p, p, p, None, p, 1, 1, 8, 8, 64, 1.0, 0, 0, 0, 3, C.addressof(st)) == 1
    # NULL strides = the packed entry
    assert lib.mhip_flash_attention_strided(None, p, p, p, None, p, 1, 1, 8, 8, 64, 1.0, 0, 0, 0, 1, None) == 0
    torch.cuda.synchronize()


def test_attention_invariants():
    from metalhlo_amd import kernels
    q, k, v = _qkv(1, 2, 256, 256, 128, torch.bfloat16, 44)
    # uniform V rows -> every output row equals that row (softmax weights sum to 1)
    vu = v[:, :, :1].expand_as(v).contiguous()
    o = kernels.flash_attention(q, k, vu, is_causal=True)
    assert_close(o, as_f64(vu), 2e-2, "uniform V")
    # causal flag == additive upper-triangular -inf mask
    m = np.where(np.arange(256)[None, :] > np.arange(256)[:, None], -np.inf, 0.0)[None, None]
    a = kernels.flash_attention(q, k, v, is_causal=True)
    b = kernels.flash_attention(q, k, v, mask=to_dev(m, torch.bfloat16))
    assert_close(a, as_f64(b), 2e-2, "causal == mask")
    # one dominant key: q.k huge for key 7 -> output ~ V[7]
    kk = k.clone(); kk[:, :, 7] = q[:, :, 0] * 8
    o = kernels.flash_attention(q, kk, v, scale=1.0)
    assert_close(o[:, :, 0], as_f64(v[:, :, 7]), 2e-2, "dominant key")


@pytest.mark.parametrize("causal,S", [(True, 4096), (False, 2048)], ids=["causal4096", "full2048"])
def test_attention_baseline_shape_sampled(causal, S):
    """The attention benchmark configuration: bf16 B4 H32 D128 (seed 4). Oracle on sampled (b,h) slices and rows."""
    from metalhlo_amd import kernels
    B, H, D = 4, 32, 128
    rng = np.random.default_rng(4)
    q, k, v = (to_dev(rng.standard_normal((B, H, S, D), dtype=np.float32), torch.bfloat16) for _ in range(3))
    o = kernels.flash_attention(q, k, v, is_causal=causal)
    rows = np.r_[0, 1, 31, 32, 63, 64, 127, 128, S - 129, S - 1, rng.integers(0, S, 22)]
    for b, h in [(0, 0), (1, 7), (3, 31), (2, 16)]:
        exp = oracle.attention_rows(as_f64(q[b, h]), as_f64(k[b, h]), as_f64(v[b, h]), rows,
                                    is_causal=causal)
        assert_close(o[b, h][rows], exp, 2e-2, f"slice {(b, h)}")
    if causal:
        assert torch.equal(o[:, :, 0], v[:, :, 0])     # first causal row copies V[0] exactly
    assert torch.isfinite(o.float()).all()


def test_attention_errors(lib):
    x = torch.zeros(16, dtype=torch.float32, device="cuda")
    p = x.data_ptr()
    assert lib.mhip_flash_attention(None, None, p, p, None, p, 1, 1, 1, 1, 4, 1.0, 0, 0, 0, 1) == 1
    assert lib.mhip_flash_attention(None, p, p, p, None, p, 1, 1, 1, 1, 512, 1.0, 0, 0, 0, 1) == 2
    assert lib.mhip_flash_attention(None, p, p, p, None, p, 0, 1, 1, 1, 4, 1.0, 0, 0, 0, 1) == 0
    assert lib.mhip_flash_attention(None, p, p, p, None, p, 1, 1, 1, 1, 4, 1.0, 0, 0, 0, 7) == 2
