"""Writes tests/golden/interpret.json: the single-operation cases of the StableHLO
interpreter conformance files the reference keeps under
Tests/MetalHLOTests/Conformance/StableHLO/interpret/ (its StableHLOConformanceTests run
them), for the operations the host here executes.  Each case is data: the constant
operands, the operation under test (as written in the file), and the expected constant of
its `check.expect_eq_const` / `check.expect_almost_eq_const` line.

Run where the reference tree is available:  python tests/golden/make_interpret.py [reference_root]
"""
import json
import os
import re
import sys

OPS = ["abs", "add", "broadcast_in_dim", "compare", "convert", "divide", "dot_general", "exponential", "gather", "iota",
       "log", "logistic", "maximum", "minimum", "multiply", "negate", "power", "reduce", "reshape", "rsqrt", "select",
       "slice", "sqrt", "subtract", "tanh", "transpose"]
TYPES = {"f16", "f32", "f64", "bf16", "i1", "i8", "i16", "i32", "i64", "ui8", "ui16", "ui32", "ui64"}
REL = "Tests/MetalHLOTests/Conformance/StableHLO/interpret"


def statements(body_lines):
    """Joins continuation lines: a statement runs until its (), [] and {} are balanced again
    (so a region, as in the generic form of reduce, stays inside its operation)."""
    out, cur, depth = [], None, 0
    for no, ln in body_lines:
        s = ln.strip()
        if not s or s.startswith("//"):
            continue
        if cur is None:
            cur = [no, s]
        else:
            cur[1] += " " + s
        depth += sum(s.count(c) for c in "([{") - sum(s.count(c) for c in ")]}")
        if depth <= 0 and not s.endswith(","):
            out.append(cur)
            cur, depth = None, 0
    if cur:
        out.append(cur)
    # a line that does not start a statement continues the previous one (wrapped signatures)
    merged = []
    for no, s in out:
        if merged and not re.match(r"(%[\w#:]+\s*=|check\.|func\.return|return\b)", s):
            merged[-1][1] += " " + s
        else:
            merged.append([no, s])
    return merged


def element_types(text):
    return set(re.findall(r"tensor<(?:[\d?]+x)*([A-Za-z0-9]+)>", text))


def cases_of(path, op):
    lines = open(path).read().split("\n")
    out, i = [], 0
    while i < len(lines):
        m = re.match(r"\s*func\.func @(\w+)\(\)\s*\{\s*$", lines[i])
        if not m:
            i += 1
            continue
        start, name = i, m.group(1)
        body = []
        i += 1
        while i < len(lines) and lines[i].strip() != "}":
            body.append((i + 1, lines[i]))
            i += 1
        sts = statements(body)
        consts, ops, checks, other = [], [], [], 0
        for no, s in sts:
            c = re.match(r"(%\w+) = stablehlo\.constant dense<(.*)> : (tensor<[^>]*>)$", s)
            k = re.match(r"check\.expect_(almost_)?eq_const (%\w+), dense<(.*)> : (tensor<[^>]*>)$", s)
            if c:
                consts.append([c.group(1), c.group(2), c.group(3)])
            elif k:
                checks.append([bool(k.group(1)), k.group(2), k.group(3), k.group(4)])
            elif re.match(r"(func\.return|return)$", s):
                pass
            elif re.match(r"%\w+ = \"?stablehlo\." + op + r"\b", s):
                ops.append(s)
            else:
                other += 1
        if other or len(ops) != 1 or len(checks) != 1:
            continue
        res = re.match(r"(%\w+) =", ops[0]).group(1)
        almost, target, expect, rtype = checks[0]
        if target != res:
            continue
        text = " ".join([c[2] for c in consts] + [ops[0], rtype])
        if not element_types(text) <= TYPES or "complex" in text or "!quant" in text or "0x" in " ".join(c[1] for c in consts) + expect:
            continue
        out.append(dict(src=f"{REL}/{os.path.basename(path)}:{start + 1}", name=name, consts=consts, op=ops[0], result=res,
                        result_type=rtype, expect=expect, almost=almost))
    return out


def main():
    root = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    cases = []
    for op in OPS:
        p = os.path.join(root, REL, op + ".mlir")
        if os.path.exists(p):
            cases += cases_of(p, op)
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "interpret.json")
    with open(out, "w") as f:
        json.dump(cases, f, indent=0)
    per = {}
    for c in cases:
        per[c["src"].split("/")[-1].split(".")[0]] = per.get(c["src"].split("/")[-1].split(".")[0], 0) + 1
    print(len(cases), "cases:", per)


if __name__ == "__main__":
    main()
