#!/usr/bin/env python3
"""Writes tests/golden/benchmark_modules.json: the StableHLO programs of the reference's own
benchmark suite that lie on the fused-transformer path, instantiated at the configurations its
README publishes figures for.  The programs are inputs of the system under test (MLIR text the
reference feeds to its compiler); they are taken from the string templates in

    Sources/MetalHLOBenchmarks/ModelBenchmarks.swift      (attention core, self-attention, FFN,
                                                           softmax, encoder block, MLP FFN)
    Sources/MetalHLOBenchmarks/OperationBenchmarks.swift  (LayerNorm)

by evaluating the Swift string interpolations for the chosen configuration.  Each entry records
the benchmark id, the file and line of its template, the argument shapes with the distribution
the reference's input generator uses, and the figure the reference publishes (README.md).

Run in the build container (the reference is mounted at /root/reference):
    python tests/golden/make_benchmark_modules.py
"""
import json
import math
import os
import re
import textwrap

REF = os.environ.get("METALHLO_REFERENCE", "/root/reference")
HERE = os.path.dirname(os.path.abspath(__file__))
MODEL = "Sources/MetalHLOBenchmarks/ModelBenchmarks.swift"
OPS = "Sources/MetalHLOBenchmarks/OperationBenchmarks.swift"


def read(rel):
    with open(os.path.join(REF, rel)) as f:
        return f.read()


def line_of(text, pos):
    return text.count("\n", 0, pos) + 1


def triple_quoted(text, start):
    """The first \"\"\" ... \"\"\" literal at or after `start`: (content, position)."""
    a = text.index('"""', start)
    b = text.index('"""', a + 3)
    return textwrap.dedent(text[a + 3:b]).strip("\n"), a


def interpolate(template, env):
    def sub(m):
        expr = m.group(1).strip()
        if expr not in env:
            raise KeyError(f"no value for \\({expr})")
        return str(env[expr])
    return re.sub(r"\\\(([^()]*)\)", sub, template)


def swift_double(x):
    """How Swift prints a Double in a string interpolation (shortest round-trip form)."""
    r = repr(float(x))
    return r if "e" not in r else r.replace("e-0", "e-").replace("e+0", "e+")


def static_module(text, bench_id):
    pos = text.index(f'id: "{bench_id}"')
    prog = text.index("mlirProgram:", pos)
    body, at = triple_quoted(text, prog)
    return body, line_of(text, at)


def attention_core(text, B, H, S, D):
    pos = text.index("private static func attentionCoreMLIR")
    end = text.index("return \"\"\"", pos)
    env = {"B": B, "H": H, "S": S, "D": D, "scale": swift_double(1.0 / math.sqrt(D))}
    for m in re.finditer(r'let (\w+) = "([^"\n]*)"', text[pos:end]):
        env[m.group(1)] = interpolate(m.group(2), env)
    body, at = triple_quoted(text, end)
    return interpolate(body, env), line_of(text, at)


def layer_norm(text, bench_id, batch, seq, hidden):
    pos = text.index("let layerNormConfigs")
    body, at = triple_quoted(text, text.index("let mlir =", pos))
    env = {"config.batch": batch, "config.seq": seq, "config.hidden": hidden,
           "moduleId": bench_id.replace("-", "_"), "hiddenFloat": swift_double(float(hidden))}
    return interpolate(body, env), line_of(text, at)


def main():
    model, ops = read(MODEL), read(OPS)
    out = []

    def add(bench_id, name, mlir, src, line, inputs, published):
        out.append(dict(id=bench_id, name=name, source=f"{src}:{line}", inputs=inputs, published=published, mlir=mlir))

    U = lambda shape, lo=-1.0, hi=1.0: dict(shape=shape, dist="uniform", lo=lo, hi=hi)
    N = lambda shape, std=1.0: dict(shape=shape, dist="normal", mean=0.0, std=std)
    Z = lambda shape: dict(shape=shape, dist="zeros")

    mlir, ln = attention_core(model, 8, 12, 128, 64)
    add("ATTN-002", "Attention core B8 H12 S128 D64", mlir, MODEL, ln, [N([8, 12, 128, 64])] * 3,
        "0.65 ms, Apple M5 Pro, O3 (README.md:1203)")
    for bid, b, s, h, pub in (("NORM-LN-002", 32, 128, 768, "4.42 / 6.17 / 6.87 / 6.46 ms, Apple M1; 1.42 ms, M5 Pro (README.md:1126,1204)"),
                              ("NORM-LN-004", 8, 2048, 768, "15.67 / 20.90 / 21.10 / 23.02 ms, Apple M1 (README.md:1128)")):
        mlir, ln = layer_norm(ops, bid, b, s, h)
        add(bid, f"LayerNorm {b}x{s}x{h}", mlir, OPS, ln, [U([b, s, h], 0.0, 1.0), U([h], 0.8, 1.2), U([h], -0.1, 0.1)], pub)
    w = lambda *s: N(list(s), 0.02)
    static = [
        ("XFMR-INF-001", "Self-attention seq 128, hidden 768, 12 heads, batch 1",
         [U([1, 128, 768], 0.0, 1.0), w(768, 768), w(768, 768), w(768, 768), w(768, 768)],
         "2.76 / 2.51 / 2.19 / 2.41 ms, Apple M1 (README.md:1136)"),
        ("XFMR-INF-004", "Transformer FFN 768 -> 3072 -> 768, batch 8, seq 128",
         [U([8, 128, 768], 0.0, 1.0), w(768, 3072), Z([3072]), w(3072, 768), Z([768])],
         "11.27 / 18.24 / 16.71 / 16.02 ms, Apple M1 (README.md:1139)"),
        ("XFMR-INF-005", "Softmax 8x12x128x128", [U([8, 12, 128, 128], -5.0, 5.0)],
         "2.53 / 2.34 / 2.29 / 2.29 ms, Apple M1 (README.md:1140)"),
        ("XFMR-INF-006", "Transformer encoder block, batch 1, seq 128", None,
         "7.71 / 7.46 / 8.48 / 7.84 ms, Apple M1 (README.md:1141)"),
    ]
    for bid, name, inputs, pub in static:
        mlir, ln = static_module(model, bid)
        if inputs is None:      # argument shapes from the signature; weights N(0, 0.02), the rest uniform / ones / zeros by name
            sig = mlir[mlir.index("@main(") + 6:mlir.index(") ->")]
            inputs = []
            for nm, shape in re.findall(r"%(\w+): tensor<([0-9x]+)xf32>", sig):
                dims = [int(d) for d in shape.split("x")]
                inputs.append(U(dims, 0.0, 1.0) if nm == "x" else U(dims, 0.8, 1.2) if nm.endswith("_g") else
                              Z(dims) if nm.endswith("_b") or nm.startswith("ff_b") else N(dims, 0.02))
        add(bid, name, mlir, MODEL, ln, inputs, pub)
    path = os.path.join(HERE, "benchmark_modules.json")
    with open(path, "w") as f:
        json.dump(out, f, indent=1)
    print(f"wrote {len(out)} modules to {path} ({os.path.getsize(path)} bytes)")


if __name__ == "__main__":
    main()
