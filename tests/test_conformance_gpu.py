"""GPU: the single-operation cases of the StableHLO interpreter conformance files the reference
keeps (tests/golden/interpret.json, written by tests/golden/make_interpret.py) run through
the mhlo_* C API: constants in, one operation, the file's expected constant out.
Integer, index and boolean results must be bit-exact; floating point within 1e-5 (f32 / f64)
or 2e-2 (16-bit) by the rule |got - e| <= max(tol, tol * |e|)."""
import json
import os
import re

import numpy as np
import pytest

from oracle import oracle

pytestmark = pytest.mark.gpu

CASES = json.load(open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "interpret.json")))
# operations of these files the host does not execute in the form the case uses
UNSUPPORTED = (4, "MHLO_ERROR_UNSUPPORTED_OP")


@pytest.fixture(scope="module")
def sess():
    from metalhlo_amd import capi
    s = capi.Session()
    yield s
    s.close()


NP = {"i1": np.bool_, "i8": np.int8, "i16": np.int16, "i32": np.int32, "i64": np.int64, "ui8": np.uint8, "ui16": np.uint16,
      "ui32": np.uint32, "ui64": np.uint64}


def parse_literal(text, shape, et):
    """dense<...> payload -> numpy array of `shape`: float64 for the floating types, the exact
    integer / boolean type otherwise (Python integers, so 64-bit values keep every bit)."""
    toks = re.findall(r"true|false|[-+]?(?:inf|nan|\d+\.?\d*(?:[eE][-+]?\d+)?|\.\d+(?:[eE][-+]?\d+)?)",
                      text.replace("INF", "inf").replace("NaN", "nan"))
    if et in NP:
        vals = [{"true": 1, "false": 0}[t] if t in ("true", "false") else int(t) for t in toks]
    else:
        vals = [float(t) for t in toks]
    n = int(np.prod(shape)) if shape else 1
    if len(vals) == 1 and n != 1:
        vals = vals * n                                   # splat
    assert len(vals) == n, (text, shape)
    return np.array(vals, dtype=NP.get(et, np.float64)).reshape(shape)


def tensor_type(t):
    m = re.match(r"tensor<((?:\d+x)*)([a-z]+\d*)>", t)
    shape = [int(d) for d in m.group(1).split("x") if d]
    return shape, m.group(2)


def to_f64(arr, et):
    if et == "bf16":
        return oracle.bf16_bits_to_f32(arr).astype(np.float64)
    return np.asarray(arr).astype(np.float64)


@pytest.mark.parametrize("case", CASES, ids=lambda c: c["src"].split("/")[-1].replace(".mlir", "") + "-" + c["name"])
def test_interpret_case(case, sess):
    from metalhlo_amd import capi
    body = "\n".join(f"    {n} = stablehlo.constant dense<{lit}> : {t}" for n, lit, t in case["consts"])
    text = (f"module {{\n  func.func @main() -> ({case['result_type']}) {{\n{body}\n    {case['op']}\n"
            f"    return {case['result']} : {case['result_type']}\n  }}\n}}\n")
    try:
        exe = sess.compile(text)
    except capi.MHLOError as e:
        if e.code == UNSUPPORTED[0]:
            pytest.skip(f"form not executed by the host: {e}")
        raise
    got = sess.run(exe, [])[0]
    sess.lib.mhlo_executable_destroy(exe)
    shape, et = tensor_type(case["result_type"])
    exp = parse_literal(case["expect"], shape, et)
    assert list(np.asarray(got).shape) == shape
    g = to_f64(got, et)
    if et in ("f16", "bf16", "f32", "f64"):
        tol = 2e-2 if et in ("f16", "bf16") else 1e-5
        bad = ~(np.abs(g - exp) <= np.maximum(tol, tol * np.abs(exp)))
        bad &= ~(np.isnan(g) & np.isnan(exp)) & ~((g == exp))          # equal infinities / both NaN are fine
        assert not bad.any(), (g, exp)
    else:
        got = np.asarray(got)
        if et == "i1":                                     # one byte per element on the device, 0 or 1
            assert got.dtype == np.uint8 and got.max(initial=0) <= 1, got
            got = got.astype(np.bool_)
        assert got.dtype == exp.dtype and np.array_equal(got, exp), (got, exp)


def test_most_cases_are_executed(sess):
    """The skip above is for forms outside the operator subset, not a way to hide failures:
    all 135 cases must compile."""
    from metalhlo_amd import capi
    ok = 0
    for case in CASES:
        body = "\n".join(f"    {n} = stablehlo.constant dense<{lit}> : {t}" for n, lit, t in case["consts"])
        text = (f"module {{\n  func.func @main() -> ({case['result_type']}) {{\n{body}\n    {case['op']}\n"
                f"    return {case['result']} : {case['result_type']}\n  }}\n}}\n")
        try:
            sess.lib.mhlo_executable_destroy(sess.compile(text))
            ok += 1
        except capi.MHLOError:
            pass
    assert len(CASES) == 135 and ok == 135, (len(CASES), ok)


def spec_gather(x, idx, offset_dims, collapsed, start_index_map, ivd, slice_sizes, op_batching=(), idx_batching=()):
    """stablehlo.gather by the specification's index arithmetic, one result element at a time."""
    idx_dims = [d for d in range(idx.ndim) if d != ivd]
    kept = [d for d in range(x.ndim) if d not in collapsed and d not in op_batching]
    rank = len(idx_dims) + len(offset_dims)
    shape, bi, oi = [], 0, 0
    for r in range(rank):
        if r in offset_dims:
            shape.append(slice_sizes[kept[oi]]); oi += 1
        else:
            shape.append(idx.shape[idx_dims[bi]]); bi += 1
    out = np.zeros(shape, dtype=x.dtype)
    for ri in np.ndindex(*shape):
        batch = [ri[r] for r in range(rank) if r not in offset_dims]
        offs = [ri[r] for r in range(rank) if r in offset_dims]
        sel = list(batch)
        if ivd < idx.ndim:
            sel.insert(ivd, slice(None))
        start = np.atleast_1d(idx[tuple(sel)])
        full = [0] * x.ndim
        for c, d in enumerate(start_index_map):
            full[d] = int(np.clip(start[c], 0, x.shape[d] - slice_sizes[d]))
        for ob, ib in zip(op_batching, idx_batching):
            full[ob] = batch[ib - (0 if ib < ivd else 1)]
        for k, d in enumerate(kept):
            full[d] += offs[k]
        out[ri] = x[tuple(full)]
    return out


GATHER_FORMS = [
    # operand shape, indices shape, offset_dims, collapsed, start_index_map, index_vector_dim, slice_sizes, batching
    ((3, 4, 2), (2, 3, 2), [2, 3], [0], [1, 0], 2, [1, 2, 2], [], []),            # the reference file's first case
    ((2, 3, 4, 2), (2, 2, 3, 2), [3, 4], [1], [2, 1], 3, [1, 1, 2, 2], [0], [1]),  # ... and its batching case
    ((7, 5), (6,), [1], [0], [0], 1, [1, 5], [], []),                              # rows, index_vector_dim == rank
    ((7, 5), (6, 1), [1], [0], [0], 1, [1, 5], [], []),                            # rows, explicit vector of one
    ((7, 5), (4, 2), [], [0, 1], [0, 1], 1, [1, 1], [], []),                       # element picks (gather_nd)
    ((7, 5), (2, 4), [0, 1], [], [1, 0], 0, [3, 2], [], []),                       # windows, index vector first
    ((5, 6, 3), (4, 1), [0, 2], [1], [1], 1, [5, 1, 2], [], []),                   # column picks with a narrowed last dim
]


@pytest.mark.parametrize("form", GATHER_FORMS, ids=[str(i) for i in range(len(GATHER_FORMS))])
@pytest.mark.parametrize("types", [("f32", "i64"), ("i64", "i32"), ("bf16", "i32"), ("i8", "i64")])
def test_gather_forms(form, types, sess):
    """General gather through the C API against the specification's arithmetic; indices reach outside
    the operand on both sides, so the clamp to [0, dim - slice_size] is exercised."""
    xs, ishape, offset_dims, collapsed, sim, ivd, slices, ob, ib = form
    et, it = types
    rng = np.random.default_rng(len(xs) * 100 + len(ishape) + ivd)
    np_et = {"f32": np.float32, "i64": np.int64, "bf16": np.uint16, "i8": np.int8}[et]
    x = rng.integers(-100, 100, xs).astype(np_et) if et != "bf16" else rng.integers(0, 2 ** 15, xs).astype(np.uint16)
    idx = rng.integers(-2, max(xs) + 2, ishape).astype({"i32": np.int32, "i64": np.int64}[it])
    exp = spec_gather(x, idx, offset_dims, collapsed, sim, ivd, slices, ob, ib)
    tt = lambda shape, e: "tensor<" + "".join(f"{d}x" for d in shape) + e + ">"
    batching = (f"operand_batching_dims = {ob}, start_indices_batching_dims = {ib}, " if ob else "")
    text = (f"module {{\n  func.func @main(%operand: {tt(xs, et)}, %start_indices: {tt(ishape, it)}) -> ({tt(exp.shape, et)}) {{\n"
            f'    %result = "stablehlo.gather"(%operand, %start_indices) {{ dimension_numbers = #stablehlo.gather< '
            f"offset_dims = {offset_dims}, collapsed_slice_dims = {collapsed}, {batching}start_index_map = {sim}, "
            f"index_vector_dim = {ivd}>, slice_sizes = array<i64: {', '.join(map(str, slices))}>, indices_are_sorted = false }} "
            f": ({tt(xs, et)}, {tt(ishape, it)}) -> {tt(exp.shape, et)}\n"
            f"    return %result : {tt(exp.shape, et)}\n  }}\n}}\n")
    exe = sess.compile(text)
    got = np.asarray(sess.run(exe, [(x, et), (idx, it)])[0])
    sess.lib.mhlo_executable_destroy(exe)
    assert got.shape == exp.shape and np.array_equal(got.view(exp.dtype) if got.dtype != exp.dtype else got, exp)


def test_spec_gather_reproduces_the_reference_cases():
    """Pins the checker above: it reproduces the two gather cases of the reference's file."""
    seen = 0
    for case in CASES:
        if "gather.mlir" not in case["src"]:
            continue
        dn = case["op"]
        ints = lambda key: [int(v) for v in re.search(key + r" = \[([\d, ]*)\]", dn).group(1).replace(" ", "").split(",") if v]
        opt = lambda key: ints(key) if re.search(r"\b" + key + r" = \[", dn) else []
        slices = [int(v) for v in re.search(r"slice_sizes = array<i64: ([\d, ]+)>", dn).group(1).split(",")]
        ivd = int(re.search(r"index_vector_dim = (\d+)", dn).group(1))
        (xn, xl, xt), (inn, il, itt) = case["consts"]
        x = parse_literal(xl, *tensor_type(xt))
        idx = parse_literal(il, *tensor_type(itt))
        exp = parse_literal(case["expect"], *tensor_type(case["result_type"]))
        got = spec_gather(x, idx, ints("offset_dims"), ints("collapsed_slice_dims"), ints("start_index_map"), ivd, slices,
                          opt("operand_batching_dims"), opt("start_indices_batching_dims"))
        assert np.array_equal(got, exp), case["name"]
        seen += 1
    assert seen == 2
