"""GPU parity: glue operators. Integer / index / copy results must be bit-exact."""
import numpy as np
import pytest
import torch

from oracle import oracle
from tests.util import as_f64, assert_close, to_dev

pytestmark = pytest.mark.gpu


def test_gather_rows_bit_exact_and_clamp():
    from metalhlo_amd import kernels
    rng = np.random.default_rng(51)
    for dtype, width in [(torch.float32, 768), (torch.bfloat16, 768), (torch.float32, 5), (torch.int64, 3)]:
        tab = torch.from_numpy(rng.integers(-1000, 1000, (97, width))).to(dtype).cuda()
        for idt in (torch.int32, torch.int64):
            idx = torch.from_numpy(rng.integers(-3, 101, (4, 9))).to(idt).cuda()   # some out of range
            out = kernels.gather_rows(tab, idx)
            exp = tab[idx.long().clamp(0, 96)]
            assert out.shape == (4, 9, width) and torch.equal(out, exp)


def test_embed_tokens():
    from metalhlo_amd import kernels
    rng = np.random.default_rng(52)
    wte = to_dev(rng.standard_normal((503, 96)) * 0.02, torch.float32)
    wpe = to_dev(rng.standard_normal((64, 96)) * 0.02, torch.float32)
    ids = torch.from_numpy(rng.integers(0, 503, (3, 40)).astype(np.int32)).cuda()
    out = kernels.embed_tokens(ids, wte, wpe, torch.bfloat16)
    s = as_f64(wte)[ids.cpu().numpy()] + as_f64(wpe)[None, :40]
    exp_bits = oracle.bf16_round_bits(s.astype(np.float32))       # fp32 sum, one RNE rounding
    got_bits = out.cpu().view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(got_bits, exp_bits)
    out32 = kernels.embed_tokens(ids, wte, wpe, torch.float32)
    assert np.array_equal(out32.cpu().numpy(), s.astype(np.float32))


def test_add_and_convert():
    from metalhlo_amd import kernels
    rng = np.random.default_rng(53)
    for n in (1, 7, 4096, 100003):
        a = to_dev(rng.standard_normal(n), torch.bfloat16)
        b = to_dev(rng.standard_normal(n), torch.bfloat16)
        got = kernels.add(a, b).cpu().view(torch.int16).numpy().view(np.uint16)
        exp = oracle.bf16_round_bits((as_f64(a) + as_f64(b)).astype(np.float32))
        assert np.array_equal(got, exp)
        ai = torch.from_numpy(rng.integers(-2**31, 2**31 - 1, n).astype(np.int32)).cuda()
        bi = torch.from_numpy(rng.integers(-2**31, 2**31 - 1, n).astype(np.int32)).cuda()
        assert torch.equal(kernels.add(ai, bi), ai + bi)      # wraps
    x = to_dev(rng.standard_normal(10001) * 100, torch.float32)
    got = kernels.convert(x, torch.bfloat16).cpu().view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(got, oracle.bf16_round_bits(x.cpu().numpy()))
    # ties-to-even and NaN
    ties = torch.tensor([1.00390625, 1.01171875, float("nan"), float("inf"), -0.0], dtype=torch.float32).cuda()
    got = kernels.convert(ties, torch.bfloat16).cpu().view(torch.int16).numpy().view(np.uint16)
    exp = oracle.bf16_round_bits(ties.cpu().numpy())
    assert np.array_equal(got[[0, 1, 3, 4]], exp[[0, 1, 3, 4]]) and (got[2] & 0x7F80) == 0x7F80 and (got[2] & 0x7F)
    back = kernels.convert(kernels.convert(x, torch.bfloat16), torch.float32)
    assert np.array_equal(back.cpu().numpy(), oracle.bf16_bits_to_f32(oracle.bf16_round_bits(x.cpu().numpy())))
    xi = torch.from_numpy(rng.integers(-10**6, 10**6, 999).astype(np.int32)).cuda()
    assert torch.equal(kernels.convert(xi, torch.float32), xi.float())
    assert torch.equal(kernels.convert(xi, torch.int64), xi.long())
    xf = to_dev(rng.standard_normal(999) * 1000, torch.float32)
    assert torch.equal(kernels.convert(xf, torch.int32), xf.to(torch.int32))   # truncation toward zero


def test_transposes_and_iota():
    from metalhlo_amd import kernels
    rng = np.random.default_rng(54)
    x = to_dev(rng.standard_normal((2, 5, 3, 16)), torch.bfloat16)
    assert torch.equal(kernels.transpose_0213(x), x.permute(0, 2, 1, 3).contiguous())
    xf = to_dev(rng.standard_normal((3, 4, 7, 5)), torch.float32)
    assert torch.equal(kernels.transpose_0213(xf), xf.permute(0, 2, 1, 3).contiguous())
    qkv = to_dev(rng.standard_normal((2, 33, 3 * 4 * 64)), torch.bfloat16)
    q, k, v = kernels.split_qkv_heads(qkv, 4)
    for got, part in zip((q, k, v), qkv.split(4 * 64, dim=-1)):
        assert torch.equal(got, part.reshape(2, 33, 4, 64).permute(0, 2, 1, 3).contiguous())
    for dt in (torch.int32, torch.int64, torch.float32, torch.uint8):
        for dim in range(3):
            y = kernels.iota((3, 5, 4), dim, dt)
            shape = [1, 1, 1]; shape[dim] = -1
            exp = torch.arange((3, 5, 4)[dim]).reshape(shape).expand(3, 5, 4).to(dt)
            assert torch.equal(y.cpu(), exp)


def test_argmax_ties_and_nan():
    from metalhlo_amd import kernels
    rng = np.random.default_rng(55)
    x = rng.integers(0, 50, (37, 1000)).astype(np.float32)          # many ties
    x[3, 10] = x[3, 500] = 99.0
    x[4, 77] = np.nan; x[4, 900] = np.nan
    x[5, :] = -np.inf
    xd = torch.from_numpy(x).cuda()
    idx, val = kernels.argmax(xd, return_values=True)
    exp = np.array([int(np.flatnonzero(np.isnan(r))[0]) if np.isnan(r).any() else int(np.argmax(r)) for r in x])
    assert np.array_equal(idx.cpu().numpy(), exp.astype(np.int32))
    assert idx[3].item() == 10 and idx[4].item() == 77 and idx[5].item() == 0
    assert np.array_equal(val.cpu().numpy()[[0, 3]], x[[0, 3], exp[[0, 3]]])
    i64 = kernels.argmax(xd.to(torch.bfloat16), index_dtype=torch.int64)
    xb = xd.to(torch.bfloat16).float().cpu().numpy()
    exp_b = np.array([int(np.flatnonzero(np.isnan(r))[0]) if np.isnan(r).any() else int(np.argmax(r)) for r in xb])
    assert np.array_equal(i64.cpu().numpy(), exp_b)
    # vocab-sized row
    big = torch.from_numpy(rng.standard_normal((8, 50257)).astype(np.float32)).cuda()
    assert torch.equal(kernels.argmax(big).long(), big.argmax(-1))


def test_convert_batch_matches_single_converts(lib):
    """Many tensors in one launch: same bits as one mhip_convert each (and as torch's rounding), for
    sizes around the 8-element vectors and the 2048-element blocks, unaligned bases, empty
    tensors, and more tensors than one launch's table holds."""
    import ctypes as C
    rng = np.random.default_rng(91)
    sizes = [1, 7, 8, 9, 2047, 2048, 2049, 0, 768, 3 * 768, 768 * 768, 5] + [int(v) for v in rng.integers(1, 5000, 120)]
    for dst, code in ((torch.bfloat16, 3), (torch.float16, 0)):
        big = torch.from_numpy(rng.standard_normal(sum(sizes) + 16 * len(sizes) + 64).astype(np.float32)).cuda()
        outs_flat = torch.full((big.numel(),), 9.0, dtype=dst, device="cuda")
        xs, ys, off = [], [], 0
        for i, n in enumerate(sizes):
            off += (i % 4)                                   # every alignment of the base modulo 4 elements
            xs.append(big[off:off + n])
            ys.append(outs_flat[off:off + n])
            off += n + 8
        px = (C.c_void_p * len(sizes))(*[x.data_ptr() for x in xs])
        py = (C.c_void_p * len(sizes))(*[y.data_ptr() for y in ys])
        pn = (C.c_int64 * len(sizes))(*sizes)
        assert lib.mhip_convert_batch(None, len(sizes), px, py, pn, 1, code) == 0, lib.mhip_last_error()
        torch.cuda.synchronize()
        want = torch.full_like(outs_flat, 9.0)
        off = 0
        for i, n in enumerate(sizes):
            off += (i % 4)
            want[off:off + n] = big[off:off + n].to(dst)
            off += n + 8
        assert torch.equal(outs_flat, want)                  # converted where asked, untouched elsewhere
    assert lib.mhip_convert_batch(None, 1, px, py, pn, 3, 1) == 2      # only f32 -> 16-bit
    assert lib.mhip_convert_batch(None, 0, None, None, None, 1, 3) == 0
