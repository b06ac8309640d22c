"""Writes tests/golden/kat.json: the known-answer values the reference's own
tests hold for the fused-kernel path (inputs and expected outputs only).

Where the reference test computes its expectation from a closed form at run time
(softmax, GELU) the same closed form is evaluated here with Python's ``math``
module, independently of oracle/oracle.py, so that the oracle can be checked
against this file.  Run: ``python tests/golden/make_kat.py``.
Citations are relative to the reference tree.
"""
import json
import math
import os


def softmax_row(r):
    m = max(r)
    e = [math.exp(v - m) for v in r]
    s = sum(e)
    return [v / s for v in e]


def gelu_tanh(x):
    return 0.5 * x * (1 + math.tanh(0.7978845608 * (x + 0.044715 * x * x * x)))


def ln_row(r, eps):
    n = len(r)
    mu = sum(r) / n
    var = sum((v - mu) ** 2 for v in r) / n
    return [(v - mu) / math.sqrt(var + eps) for v in r]


kat = {
    "softmax": [
        {"src": "Tests/MetalHLOTests/ActivationOpsTests.swift:137-192", "x": [[1, 2, 3, 4]],
         "y": [softmax_row([1, 2, 3, 4])], "tol": 1e-5},
        {"src": "Tests/MetalHLOCoreTests/MetalKernelTests.swift:89-101", "x": [[0, 0, 0, 0]],
         "y": [[0.25, 0.25, 0.25, 0.25]], "tol": 1e-5},
        {"src": "Examples/JAXExample/jax_metalhlo_example.py:377-382",
         "x": [[1, 2, 3, 4], [1, 1, 1, 1]],
         "y": [softmax_row([1, 2, 3, 4]), [0.25, 0.25, 0.25, 0.25]], "tol": 1e-5},
    ],
    "gelu": [
        {"src": "Tests/MetalHLOTests/ActivationOpsTests.swift:252-318", "x": [-2, -1, 0, 1, 2, 3],
         "y": [gelu_tanh(v) for v in (-2, -1, 0, 1, 2, 3)], "tol": 1e-4},
    ],
    "rms_norm": [
        {"src": "Tests/MetalHLOCoreTests/MetalKernelTests.swift:239-274", "x": [[3, 4, 0, 0]],
         "gamma": [1, 1, 1, 1], "eps": 1e-5, "y": [[1.2, 1.6, 0, 0]], "tol": 1e-4},
    ],
    "layer_norm": [
        # the reference asserts mean ~ 0 and std ~ 1 per row at 1e-4
        {"src": "Tests/MetalHLOCoreTests/MetalKernelTests.swift:173-226",
         "x": [[1, 2, 3, 4], [10, 20, 30, 40]], "gamma": [1, 1, 1, 1], "beta": [0, 0, 0, 0],
         "eps": 1e-5, "tol": 1e-4},
        {"src": "Examples/JAXExample/jax_metalhlo_example.py:385-398",
         "x": [[1, 2, 3, 4], [2, 4, 6, 8]], "gamma": [1, 1, 1, 1], "beta": [0, 0, 0, 0],
         "eps": 1e-5, "y": [ln_row([1, 2, 3, 4], 1e-5), ln_row([2, 4, 6, 8], 1e-5)], "tol": 1e-4},
    ],
    "dot": [
        {"src": "Tests/MetalHLOTests/OperationTests.swift:327-349",
         "lhs": [[1, 2, 3], [4, 5, 6]], "rhs": [[1, 2], [3, 4], [5, 6]],
         "lhs_batch": [], "rhs_batch": [], "lhs_contract": [1], "rhs_contract": [0],
         "y": [[22, 28], [49, 64]], "tol": 0},
        {"src": "Tests/MetalHLOTests/TrainingOpsTests.swift:14-84",
         "lhs": [[[1, 0, 0, 0], [0, 1, 0, 0], [0, 0, 1, 0]],
                 [[1, 1, 1, 1], [2, 2, 2, 2], [3, 3, 3, 3]]],
         "rhs": [[[1, 0, 0, 0, 0], [0, 1, 0, 0, 0], [0, 0, 1, 0, 0], [0, 0, 0, 1, 0]],
                 [[1, 1, 1, 1, 0], [1, 1, 1, 1, 0], [1, 1, 1, 1, 0], [1, 1, 1, 1, 0]]],
         "lhs_batch": [0], "rhs_batch": [0], "lhs_contract": [2], "rhs_contract": [1],
         "y": [[[1, 0, 0, 0, 0], [0, 1, 0, 0, 0], [0, 0, 1, 0, 0]],
               [[4, 4, 4, 4, 0], [8, 8, 8, 8, 0], [12, 12, 12, 12, 0]]], "tol": 1e-5},
        {"src": "Tests/MetalHLOTests/TrainingOpsTests.swift:86-139",
         "lhs": [[1, 5, 9], [2, 6, 10], [3, 7, 11], [4, 8, 12]],
         "rhs": [[1, 1, 1, 1]] * 5,
         "lhs_batch": [], "rhs_batch": [], "lhs_contract": [0], "rhs_contract": [1],
         "y": [[10] * 5, [26] * 5, [42] * 5], "tol": 1e-5},
        # Conformance/StableHLO/interpret/dot_general.mlir (i64 cases, exact)
        {"src": "Tests/MetalHLOTests/Conformance/StableHLO/interpret/dot_general.mlir:3-16",
         "lhs": [[[1, 2], [3, 4]], [[5, 6], [7, 8]]], "rhs": [[[1, 0], [0, 1]], [[1, 0], [0, 1]]],
         "lhs_batch": [0], "rhs_batch": [0], "lhs_contract": [2], "rhs_contract": [1],
         "y": [[[1, 2], [3, 4]], [[5, 6], [7, 8]]], "tol": 0},
        {"src": "Tests/MetalHLOTests/Conformance/StableHLO/interpret/dot_general.mlir:45-60",
         "lhs": [[1, 2], [3, 4]], "rhs": [[1, 0], [0, 1]],
         "lhs_batch": [], "rhs_batch": [], "lhs_contract": [], "rhs_contract": [],
         "y": [[[[1, 0], [0, 1]], [[2, 0], [0, 2]]], [[[3, 0], [0, 3]], [[4, 0], [0, 4]]]], "tol": 0},
    ],
}

# a few digits the closed forms above must reproduce (guards the generator itself)
assert abs(kat["softmax"][0]["y"][0][3] - 0.6439142598879722) < 1e-12
assert abs(kat["gelu"][0]["y"][3] - 0.8411919906) < 1e-6
assert abs(kat["layer_norm"][1]["y"][0][0] + 1.3416354) < 1e-5

if __name__ == "__main__":
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "kat.json")
    with open(out, "w") as f:
        json.dump(kat, f, indent=1)
    print("wrote", out)
