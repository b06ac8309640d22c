"""GPU parity: the unfused StableHLO glue entries (unary / binary / compare / select /
strided copy / reduce / fill) called through the C-ABI.  Floats: fp32 1e-5, 16-bit 2e-2;
integer, predicate and copy results bit-exact."""
import ctypes as C
import math

import numpy as np
import pytest
import torch

from tests.util import as_f64, assert_close, to_dev, TOL

pytestmark = pytest.mark.gpu

DT = {torch.float16: 0, torch.float32: 1, torch.bfloat16: 3, torch.int32: 7, torch.int64: 8}
UN = dict(exp=0, tanh=1, rsqrt=2, sqrt=3, neg=4, logistic=5, abs=6, log=7, erf=8)
BIN = dict(add=0, sub=1, mul=2, div=3, max=4, min=5, pow=6)
CMP = dict(EQ=0, NE=1, LT=2, LE=3, GT=4, GE=5)
RED = dict(sum=0, max=1, min=2, prod=3)


def p(t):
    return C.c_void_p(t.data_ptr())


def ok(lib, rc):
    assert rc == 0, lib.mhip_last_error()
    torch.cuda.synchronize()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_unary(lib, dtype):
    rng = np.random.default_rng(71)
    erf = np.vectorize(math.erf)
    ref = dict(exp=np.exp, tanh=np.tanh, rsqrt=lambda v: 1 / np.sqrt(v), sqrt=np.sqrt, neg=np.negative,
               logistic=lambda v: 1 / (1 + np.exp(-v)), abs=np.abs, log=np.log, erf=erf)
    for n in (1, 9, 4099):
        for name, f in ref.items():
            v = rng.uniform(0.05, 4, n) if name in ("rsqrt", "sqrt", "log") else rng.uniform(-4, 4, n)
            x = to_dev(v, dtype)
            y = torch.empty_like(x)
            ok(lib, lib.mhip_unary(None, UN[name], p(x), p(y), n, DT[dtype]))
            assert_close(y, f(as_f64(x)), TOL[dtype], f"{name} n={n}")
    xi = torch.tensor([-5, 0, 7, -2**31 + 1], dtype=torch.int32).cuda()
    yi = torch.empty_like(xi)
    ok(lib, lib.mhip_unary(None, UN["neg"], p(xi), p(yi), 4, DT[torch.int32]))
    assert torch.equal(yi, -xi)
    ok(lib, lib.mhip_unary(None, UN["abs"], p(xi), p(yi), 4, DT[torch.int32]))
    assert torch.equal(yi, xi.abs())
    assert lib.mhip_unary(None, UN["exp"], p(xi), p(yi), 4, DT[torch.int32]) == 2     # unsupported
    assert lib.mhip_unary(None, 99, p(xi), p(yi), 4, DT[torch.float32]) == 1
    assert lib.mhip_unary(None, UN["exp"], None, None, 0, DT[torch.float32]) == 0     # empty


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_binary_compare_select(lib, dtype):
    rng = np.random.default_rng(72)
    n = 5003
    a, b = to_dev(rng.uniform(-3, 3, n), dtype), to_dev(rng.uniform(0.25, 3, n), dtype)
    A, B = as_f64(a), as_f64(b)
    ref = dict(add=A + B, sub=A - B, mul=A * B, div=A / B, max=np.maximum(A, B), min=np.minimum(A, B),
               pow=np.abs(A) ** B)
    for name, e in ref.items():
        lhs = a.abs() if name == "pow" else a
        y = torch.empty_like(a)
        ok(lib, lib.mhip_binary(None, BIN[name], p(lhs), p(b), p(y), n, DT[dtype]))
        assert_close(y, e, TOL[dtype], name)
    # NaN propagates through max / min
    an = a.clone(); an[3] = float("nan")
    y = torch.empty_like(a)
    ok(lib, lib.mhip_binary(None, BIN["max"], p(an), p(b), p(y), n, DT[dtype]))
    assert torch.isnan(y[3]) and not torch.isnan(y[4])
    a2 = a.clone(); a2[::3] = b[::3]
    for name, f in dict(EQ=np.equal, NE=np.not_equal, LT=np.less, LE=np.less_equal, GT=np.greater,
                        GE=np.greater_equal).items():
        m = torch.empty(n, dtype=torch.uint8, device="cuda")
        ok(lib, lib.mhip_compare(None, CMP[name], p(a2), p(b), p(m), n, DT[dtype]))
        assert np.array_equal(m.cpu().numpy(), f(as_f64(a2), B).astype(np.uint8)), name
    m = (torch.from_numpy(rng.integers(0, 2, n).astype(np.uint8))).cuda()
    y = torch.empty_like(a)
    ok(lib, lib.mhip_select(None, p(m), p(a), p(b), p(y), n, a.element_size(), 0))
    assert torch.equal(y, torch.where(m.bool(), a, b))
    one = torch.tensor([0], dtype=torch.uint8).cuda()
    ok(lib, lib.mhip_select(None, p(one), p(a), p(b), p(y), n, a.element_size(), 1))
    assert torch.equal(y, b)


def test_binary_int_wraps(lib):
    rng = np.random.default_rng(73)
    for dt, np_dt in ((torch.int32, np.int32), (torch.int64, np.int64)):
        info = np.iinfo(np_dt)
        a = torch.from_numpy(rng.integers(info.min, info.max, 1001, dtype=np_dt)).cuda()
        b = torch.from_numpy(rng.integers(info.min, info.max, 1001, dtype=np_dt)).cuda()
        y = torch.empty_like(a)
        for name, e in (("add", a + b), ("sub", a - b), ("mul", a * b), ("max", torch.maximum(a, b)),
                        ("min", torch.minimum(a, b))):
            ok(lib, lib.mhip_binary(None, BIN[name], p(a), p(b), p(y), 1001, DT[dt]))
            assert torch.equal(y, e), name
        m = torch.empty(1001, dtype=torch.uint8, device="cuda")
        ok(lib, lib.mhip_compare(None, CMP["LT"], p(a), p(b), p(m), 1001, DT[dt]))
        assert torch.equal(m.bool(), a < b)


def test_narrow_unsigned_bool_and_f64_types(lib):
    """The element types beside f32 / 16-bit floats / i32 / i64: i8, i16 and the unsigned types wrap
    like numpy's; booleans are OR / AND; f64 computes in f64; integer power follows StableHLO."""
    rng = np.random.default_rng(74)
    codes = {np.int8: 5, np.int16: 6, np.uint8: 9, np.uint16: 10, np.uint32: 11, np.uint64: 12}
    n = 777
    for np_dt, code in codes.items():
        info = np.iinfo(np_dt)
        an = rng.integers(info.min, info.max, n, dtype=np_dt, endpoint=True)
        bn = rng.integers(info.min, info.max, n, dtype=np_dt, endpoint=True)
        # torch has no arithmetic on the wider unsigned types: move bytes, compute in numpy
        a = torch.from_numpy(an.view(np.uint8)).cuda()
        b = torch.from_numpy(bn.view(np.uint8)).cuda()
        y = torch.empty_like(a)
        with np.errstate(over="ignore"):
            for name, e in (("add", an + bn), ("sub", an - bn), ("mul", an * bn), ("max", np.maximum(an, bn)),
                            ("min", np.minimum(an, bn))):
                ok(lib, lib.mhip_binary(None, BIN[name], p(a), p(b), p(y), n, code))
                assert np.array_equal(y.cpu().numpy().view(np_dt), e.astype(np_dt)), (np_dt, name)
            ok(lib, lib.mhip_unary(None, UN["neg"], p(a), p(y), n, code))
            assert np.array_equal(y.cpu().numpy().view(np_dt), (0 - an).astype(np_dt)), np_dt
            ok(lib, lib.mhip_unary(None, UN["abs"], p(a), p(y), n, code))
            assert np.array_equal(y.cpu().numpy().view(np_dt), np.abs(an).astype(np_dt)), np_dt
        m = torch.empty(n, dtype=torch.uint8, device="cuda")
        ok(lib, lib.mhip_compare(None, CMP["GE"], p(a), p(b), p(m), n, code))
        assert np.array_equal(m.cpu().numpy().astype(bool), an >= bn), np_dt
    # booleans
    a = torch.from_numpy(rng.integers(0, 2, n).astype(np.uint8)).cuda()
    b = torch.from_numpy(rng.integers(0, 2, n).astype(np.uint8)).cuda()
    y = torch.empty_like(a)
    for name, e in (("add", a | b), ("max", a | b), ("mul", a & b), ("min", a & b)):
        ok(lib, lib.mhip_binary(None, BIN[name], p(a), p(b), p(y), n, 4))
        assert torch.equal(y, e), name
    assert lib.mhip_binary(None, BIN["div"], p(a), p(b), p(y), n, 4) == 2
    # f64
    x = torch.from_numpy(rng.uniform(0.1, 3.0, n)).cuda()
    z = torch.from_numpy(rng.uniform(-2.0, 2.0, n)).cuda()
    y = torch.empty_like(x)
    for name, e in (("exp", x.exp()), ("log", x.log()), ("sqrt", x.sqrt()), ("rsqrt", x.rsqrt()), ("tanh", x.tanh()),
                    ("erf", x.erf()), ("logistic", x.sigmoid()), ("neg", -x)):
        ok(lib, lib.mhip_unary(None, UN[name], p(x), p(y), n, 2))
        assert torch.allclose(y, e, rtol=1e-13, atol=1e-13), name
    for name, e in (("add", x + z), ("div", x / z), ("pow", x ** z), ("max", torch.maximum(x, z))):
        ok(lib, lib.mhip_binary(None, BIN[name], p(x), p(z), p(y), n, 2))
        assert torch.allclose(y, e, rtol=1e-13, atol=1e-13), name
    # integer power: wrap-around products; a negative exponent gives 1 / x^|e| truncated
    base = torch.from_numpy(rng.integers(-9, 10, n)).cuda()
    e = torch.from_numpy(rng.integers(-3, 25, n)).cuda()
    y = torch.empty_like(base)
    ok(lib, lib.mhip_binary(None, BIN["pow"], p(base), p(e), p(y), n, DT[torch.int64]))
    want = []
    for bb, ee in zip(base.tolist(), e.tolist()):
        if ee < 0:
            want.append(1 if bb == 1 else ((-1) ** (-ee) if bb == -1 else 0))
        else:
            v = (bb ** ee) % (1 << 64)
            want.append(v - (1 << 64) if v >= 1 << 63 else v)
    assert y.tolist() == want


def test_convert_all_pairs(lib):
    """Every pair of the thirteen element types against numpy's conversion of values every type holds exactly."""
    np_of = {0: np.float16, 1: np.float32, 2: np.float64, 4: np.bool_, 5: np.int8, 6: np.int16, 7: np.int32, 8: np.int64,
             9: np.uint8, 10: np.uint16, 11: np.uint32, 12: np.uint64}
    vals = np.array([0, 1, 2, 0, 7, 100, 127, 0, 3, 64])
    for sc, sdt in np_of.items():
        src = vals.astype(sdt)
        x = torch.from_numpy(src.view(np.uint8).copy()).cuda()
        for dc, ddt in np_of.items():
            y = torch.zeros(len(vals) * np.dtype(ddt).itemsize, dtype=torch.uint8, device="cuda")
            ok(lib, lib.mhip_convert(None, p(x), p(y), len(vals), sc, dc))
            got = y.cpu().numpy().view(np.uint8 if ddt is np.bool_ else ddt)
            assert np.array_equal(got, src.astype(ddt).astype(got.dtype)), (sdt, ddt)
    # 64-bit integers keep every bit; negative -> unsigned wraps; f64 -> integer truncates toward zero
    big = torch.tensor([2 ** 63 - 1, -1, -2 ** 63, 2 ** 53 + 1], dtype=torch.int64, device="cuda")
    y = torch.empty_like(big)
    ok(lib, lib.mhip_convert(None, p(big), p(y), 4, 8, 12))
    assert torch.equal(y, big)
    f = torch.tensor([-2.9, 2.9, -0.5, 1e15 + 1], dtype=torch.float64, device="cuda")
    ok(lib, lib.mhip_convert(None, p(f), p(y), 4, 2, 8))
    assert y.tolist() == [-2, 2, 0, 10 ** 15 + 1]
    d = torch.empty(4, dtype=torch.float64, device="cuda")
    ok(lib, lib.mhip_convert(None, p(big), p(d), 4, 8, 2))
    assert d.tolist() == [float(2 ** 63 - 1), -1.0, float(-2 ** 63), float(2 ** 53 + 1)]


def strided(lib, x, out_shape, strides, offset=0):
    y = torch.empty(out_shape, dtype=x.dtype, device="cuda")
    sh = (C.c_int64 * len(out_shape))(*out_shape)
    st = (C.c_int64 * len(out_shape))(*strides)
    ok(lib, lib.mhip_strided_copy(None, p(x), p(y), len(out_shape), sh, st, offset, x.element_size()))
    return y


def test_strided_copy_broadcast_transpose_slice(lib):
    rng = np.random.default_rng(74)
    for dt in (torch.float32, torch.bfloat16, torch.int64, torch.uint8):
        x = torch.from_numpy(rng.integers(0, 200, (6, 5, 8))).to(dt).cuda()
        s = x.stride()
        assert torch.equal(strided(lib, x, (8, 6, 5), (s[2], s[0], s[1])), x.permute(2, 0, 1).contiguous())
        assert torch.equal(strided(lib, x, (3, 5, 4), (s[0] * 2, s[1], s[2] * 2), s[0] * 1 + 1), x[1:6:2, :, 1:8:2].contiguous())
        row = x[0, 0].contiguous()
        assert torch.equal(strided(lib, row, (7, 8), (0, 1)), row.expand(7, 8).contiguous())
        sc = x[2, 3, 4:5].contiguous()
        assert torch.equal(strided(lib, sc, (4, 3), (0, 0)), sc.expand(4, 3).contiguous())
    x = torch.arange(2 ** 8, dtype=torch.float32).cuda()
    y = strided(lib, x, (2,) * 8, tuple(2 ** i for i in range(8)))         # rank 8: full bit reversal
    assert torch.equal(y, x.reshape((2,) * 8).permute(*range(7, -1, -1)).contiguous())
    sh = (C.c_int64 * 9)(*([1] * 9))
    assert lib.mhip_strided_copy(None, p(x), p(y), 9, sh, sh, 0, 4) in (1, 2)


def test_reduce_and_fill(lib):
    rng = np.random.default_rng(75)
    for dtype in (torch.float32, torch.bfloat16):
        for outer, length, inner in ((1, 4, 1), (7, 129, 1), (3, 50, 17), (1, 5000, 1), (2, 64, 256)):
            x = to_dev(rng.uniform(-1, 1, (outer, length, inner)), dtype)
            X = as_f64(x)
            for name, e, init in (("sum", X.sum(1), 0.0), ("max", X.max(1), -math.inf), ("min", X.min(1), math.inf)):
                y = torch.empty(outer, inner, dtype=dtype, device="cuda")
                ok(lib, lib.mhip_reduce(None, RED[name], p(x), p(y), outer, length, inner, init, DT[dtype]))
                tol = TOL[dtype] * (math.sqrt(length) if name == "sum" and dtype == torch.float32 else 1)
                assert_close(y, e, tol, f"{name} {outer}x{length}x{inner}")
        x = to_dev(rng.uniform(0.9, 1.1, (5, 33, 3)), dtype)
        y = torch.empty(5, 3, dtype=dtype, device="cuda")
        ok(lib, lib.mhip_reduce(None, RED["prod"], p(x), p(y), 5, 33, 3, 1.0, DT[dtype]))
        assert_close(y, as_f64(x).prod(1), TOL[dtype] * 6, "prod")
    xi = torch.from_numpy(rng.integers(-2**40, 2**40, (4, 99, 5))).cuda()
    yi = torch.empty(4, 5, dtype=torch.int64, device="cuda")
    ok(lib, lib.mhip_reduce(None, RED["sum"], p(xi), p(yi), 4, 99, 5, 3.0, DT[torch.int64]))
    assert torch.equal(yi, xi.sum(1) + 3)
    for es, dt, pat in ((1, torch.uint8, 0xAB), (2, torch.int16, 0x3F80), (4, torch.int32, 0x7FC00001),
                        (8, torch.int64, 0x0123456789ABCDEF)):
        y = torch.zeros(1003, dtype=dt, device="cuda")
        ok(lib, lib.mhip_fill(None, p(y), 1001, pat, es))
        exp = np.zeros(1003, dtype=y.cpu().numpy().dtype)
        exp[:1001] = np.array([pat], dtype=np.uint64).view(exp.dtype)[0]
        assert np.array_equal(y.cpu().numpy(), exp)
