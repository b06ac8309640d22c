"""CPU oracle for the fused transformer kernels (TEST INFRASTRUCTURE ONLY).

This module is a checker. Only tests, the smoke entry and the benchmark's
``cpu_baseline`` leg may import it; no product code path does.

Every function restates, in NumPy float64 on the *given* (already rounded)
inputs, the mathematics of one fused operator of the reference. Results are
float64; callers round to the kernel's output type with :func:`round_to` when a
bit pattern is wanted.  Citations are relative to the reference tree.

Pinning status (which independent check guards each function; the checks live
in tests/test_oracle.py):

* bf16_round_bits   — bit formula of Runtime/BufferStorage.swift:328-344, pinned
                      against torch.bfloat16 casts over all 2^16 upper halves
                      plus tie cases.
* softmax           — reference KATs (MetalKernelTests.swift:56-102,
                      ActivationOpsTests.swift:137-192,
                      jax_metalhlo_example.py:377-382), rows-sum-to-1, shift
                      invariance, torch.softmax cross-check.
* layer_norm        — KATs MetalKernelTests.swift:173-226 and
                      jax_metalhlo_example.py:385-398, affine invariance,
                      torch.layer_norm cross-check.
* rms_norm          — KAT [3,4,0,0] -> [1.2,1.6,0,0] (MetalKernelTests.swift:239-274),
                      scale covariance.
* gelu_tanh         — points -2..3 (ActivationOpsTests.swift:252-318), torch
                      gelu(approximate='tanh') cross-check.
* dot_general       — interpret/dot_general.mlir goldens, OperationTests.swift:327-349,
                      TrainingOpsTests.swift:14-139, brute-force triple loop.
* attention         — brute force on tiny sizes, invariants (uniform V, causal
                      row 0, score-shift invariance, causal flag == -inf mask),
                      torch SDPA cross-check.  The reference holds no stored
                      attention vectors: parity with the reference's *numerics*
                      beyond these is unpinned by the reference itself.
* gpt2_forward      — composition of the above; parity unpinned by any
                      reference-held vector (the reference publishes none).
* rope              — equals the complex product (x1 + i x2) e^{i theta}, preserves
                      the norm of every rotated pair, zero angle is the identity,
                      a quarter turn gives (-x2, x1), angles add under composition.
* batch_norm        — a hand-computed 2 x 2 case; with the batch's own statistics it equals
                      layer_norm of the transposed matrix (every channel normalised over the
                      rows) and gives columns of mean beta and variance gamma^2 var / (var + eps).
* depth_attention   — the reference's own cases (DepthAttentionTests.swift:46-137: equal keys
                      give the mean of the value rows, one dominant key selects its value
                      row), equals `attention` with one head and one query row, one stored
                      row returns that row, a vector added to every key changes nothing.
* elementwise_chain — each operation against the NumPy function of its name; the
                      reference's own example add -> multiply
                      (CustomCallHandlers.swift:950-953).
"""
from __future__ import annotations

import json
import math

import numpy as np

SQRT_2_OVER_PI = 0.7978845608028654  # Metal/Kernels/GELUKernel.swift:28
GELU_COEF = 0.044715                 # Metal/Kernels/GELUKernel.swift:29


# --------------------------------------------------------------------------
# dtype helpers
# --------------------------------------------------------------------------
def bf16_round_bits(x) -> np.ndarray:
    """fp32 -> bf16 bit pattern, round-to-nearest-even, NaN -> 0x7FC0.

    Follows Runtime/BufferStorage.swift:328-344:
    ``rounded = bits + 0x7FFF + ((bits >> 16) & 1)``.
    """
    f = np.ascontiguousarray(x, dtype=np.float32)
    bits = f.view(np.uint32)
    # 32-bit arithmetic: the sum only wraps for patterns above 0xFFFF8000, which are NaNs and
    # are overwritten below
    rounded = (bits >> 16) & np.uint32(1)
    rounded += np.uint32(0x7FFF)
    rounded += bits
    rounded >>= 16
    out = rounded.astype(np.uint16)
    out[np.isnan(f)] = 0x7FC0
    return out


def bf16_bits_to_f32(bits) -> np.ndarray:
    b = np.asarray(bits, dtype=np.uint16).astype(np.uint32) << 16
    return b.view(np.float32)


def round_to(x, dtype: str) -> np.ndarray:
    """Round a float64 array to `dtype` and return it widened back to float64."""
    x = np.asarray(x, dtype=np.float64)
    if dtype == "f64":
        return x
    if dtype == "f32":
        return x.astype(np.float32).astype(np.float64)
    if dtype == "f16":
        return x.astype(np.float32).astype(np.float16).astype(np.float64)
    if dtype == "bf16":
        return bf16_bits_to_f32(bf16_round_bits(x.astype(np.float32))).astype(np.float64)
    raise ValueError(dtype)


# --------------------------------------------------------------------------
# row operators
# --------------------------------------------------------------------------
def softmax(x, axis: int = -1) -> np.ndarray:
    """y = exp(x - max) / sum(exp(x - max)) over `axis`.

    Compiler/CodeGenerator.swift:4690-4794 (axis normalisation :4690-4697),
    Metal/Kernels/SoftmaxKernel.swift:36-100.
    """
    x = np.asarray(x, dtype=np.float64)
    if axis < 0:
        axis += x.ndim
    m = np.max(x, axis=axis, keepdims=True)
    m = np.where(np.isfinite(m), m, 0.0)
    e = np.exp(x - m)
    return e / np.sum(e, axis=axis, keepdims=True)


def layer_norm(x, gamma=None, beta=None, eps: float = 1e-5) -> np.ndarray:
    """(x - mean) / sqrt(var + eps) * gamma + beta, biased variance, last axis.

    Two-pass form of Compiler/CustomCallHandlers.swift:285-346 and
    Compiler/CodeGenerator.swift:4645-4686 (the hand kernel's E[x^2]-mean^2 at
    Metal/Kernels/LayerNormKernel.swift:136-138 is algebraically the same).
    """
    x = np.asarray(x, dtype=np.float64)
    mu = x.mean(axis=-1, keepdims=True)
    var = ((x - mu) ** 2).mean(axis=-1, keepdims=True)
    y = (x - mu) / np.sqrt(var + eps)
    if gamma is not None:
        y = y * np.asarray(gamma, dtype=np.float64)
    if beta is not None:
        y = y + np.asarray(beta, dtype=np.float64)
    return y


def rms_norm(x, gamma=None, eps: float = 1e-5) -> np.ndarray:
    """x * rsqrt(mean(x^2) + eps) * gamma over the last axis.

    Metal/Kernels/LayerNormKernel.swift:439-520,
    Compiler/CustomCallHandlers.swift:353-394.
    """
    x = np.asarray(x, dtype=np.float64)
    ms = (x * x).mean(axis=-1, keepdims=True)
    y = x / np.sqrt(ms + eps)
    if gamma is not None:
        y = y * np.asarray(gamma, dtype=np.float64)
    return y


def gelu_tanh(x) -> np.ndarray:
    """0.5 x (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3))).

    Metal/Kernels/GELUKernel.swift:28-44; the fused handler always uses this
    form (Compiler/CustomCallHandlers.swift:694-707).
    """
    x = np.asarray(x, dtype=np.float64)
    inner = SQRT_2_OVER_PI * (x + GELU_COEF * x * x * x)
    return 0.5 * x * (1.0 + np.tanh(inner))


def gelu_erf(x) -> np.ndarray:
    """Exact GELU 0.5 x (1 + erf(x / sqrt 2)): the function the reference's handlers name
    "gelu_exact" (Compiler/CustomCallHandlers.swift:893-894, where it falls back to the tanh
    form for lack of an erf; this restatement is the function itself)."""
    x = np.asarray(x, dtype=np.float64)
    erf = np.vectorize(math.erf, otypes=[np.float64])
    return 0.5 * x * (1.0 + erf(x / math.sqrt(2.0)))


def bias_gelu(x, bias) -> np.ndarray:
    """gelu_tanh(x + bias[col]) — the epilogue of fused_matmul_bias_activation
    (Compiler/CodeGenerator.swift:4797-4850) applied as a stand-alone row op."""
    return gelu_tanh(np.asarray(x, dtype=np.float64) + np.asarray(bias, dtype=np.float64))


ACTIVATIONS = {
    "gelu_exact": lambda v: gelu_erf(v),
    # Compiler/IntegrationTypes.swift:328-355, CustomCallHandlers.swift:540-558
    "none": lambda v: v,
    "relu": lambda v: np.maximum(v, 0.0),
    "gelu": gelu_tanh,
    "silu": lambda v: v / (1.0 + np.exp(-v)),
    "tanh": np.tanh,
    "sigmoid": lambda v: 1.0 / (1.0 + np.exp(-v)),
}


# --------------------------------------------------------------------------
# dot_general
# --------------------------------------------------------------------------
def dot_general_dims(lhs_shape, rhs_shape, lhs_batch=(), rhs_batch=(),
                     lhs_contract=None, rhs_contract=None):
    """(M, K, N, batch) exactly as Compiler/CodeGenerator.swift:5939-5970."""
    lhs_shape, rhs_shape = list(lhs_shape), list(rhs_shape)
    if lhs_contract is None:
        lhs_contract = [len(lhs_shape) - 1]
    if rhs_contract is None:
        rhs_contract = [len(rhs_shape) - 2] if len(rhs_shape) >= 2 else [0]
    m = 1
    for i, s in enumerate(lhs_shape):
        if i not in lhs_contract and i not in lhs_batch:
            m *= s
    k = 1
    for d in lhs_contract:
        k *= lhs_shape[d]
    n = 1
    for i, s in enumerate(rhs_shape):
        if i not in rhs_contract and i not in rhs_batch:
            n *= s
    if lhs_batch:
        b = 1
        for d in lhs_batch:
            b *= lhs_shape[d]
    else:
        b = int(np.prod(lhs_shape[:-2])) if len(lhs_shape) > 2 else 1
    return m, k, n, b


def dot_general(lhs, rhs, lhs_batch=(), rhs_batch=(), lhs_contract=(), rhs_contract=(),
                dtype=np.float64) -> np.ndarray:
    """StableHLO dot_general: result dims = batch, lhs free, rhs free.

    Semantics per the StableHLO spec as exercised by
    Tests/MetalHLOTests/Conformance/StableHLO/interpret/dot_general.mlir.
    Integer dtypes stay exact (int64 arithmetic)."""
    lhs = np.asarray(lhs)
    rhs = np.asarray(rhs)
    lb, rb = list(lhs_batch), list(rhs_batch)
    lc, rc = list(lhs_contract), list(rhs_contract)
    lf = [i for i in range(lhs.ndim) if i not in lb and i not in lc]
    rf = [i for i in range(rhs.ndim) if i not in rb and i not in rc]
    a = np.transpose(lhs, lb + lf + lc).astype(dtype)
    b = np.transpose(rhs, rb + rc + rf).astype(dtype)
    bs = [lhs.shape[i] for i in lb]
    ms = [lhs.shape[i] for i in lf]
    ks = [lhs.shape[i] for i in lc]
    ns = [rhs.shape[i] for i in rf]
    B, M, K, N = (int(np.prod(v)) if v else 1 for v in (bs, ms, ks, ns))
    out = np.matmul(a.reshape(B, M, K), b.reshape(B, K, N))
    return out.reshape(bs + ms + ns)


def gemm(a, b, trans_a: bool = False, trans_b: bool = False) -> np.ndarray:
    """C[b] = op(A[b]) . op(B[b]) in float64 (mixed-precision rule of
    Compiler/CodeGenerator.swift:3544-3549: wide accumulate, one final cast)."""
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    if trans_a:
        a = np.swapaxes(a, -1, -2)
    if trans_b:
        b = np.swapaxes(b, -1, -2)
    return np.matmul(a, b)


def matmul_bias_act(x, w, bias=None, activation: str = "none",
                    trans_a: bool = False, trans_b: bool = False) -> np.ndarray:
    """act(x.w + bias[col]) — Compiler/CustomCallHandlers.swift:456-560."""
    y = gemm(x, w, trans_a, trans_b)
    if bias is not None:
        y = y + np.asarray(bias, dtype=np.float64)
    return ACTIVATIONS[activation](y)


# --------------------------------------------------------------------------
# attention
# --------------------------------------------------------------------------
def attention(q, k, v, scale=None, is_causal: bool = False, mask=None) -> np.ndarray:
    """O = softmax(scale * Q K^T + mask, causal) V with materialised scores.

    Q [B,H,Sq,D], K/V [B,H,Skv,D], optional additive mask broadcastable to
    [B,H,Sq,Skv]. Causal rule: key position > query position is masked
    (Metal/Kernels/FlashAttentionKernel.swift:545,578). A fully masked row
    yields zeros (the `l > 1e-10 ? 1/l : 0` guard at :608). Default scale is
    1/sqrt(D) (FlashAttentionKernel.swift:55).
    """
    q = np.asarray(q, dtype=np.float64)
    k = np.asarray(k, dtype=np.float64)
    v = np.asarray(v, dtype=np.float64)
    d = q.shape[-1]
    if scale is None:
        scale = 1.0 / math.sqrt(d)
    s = np.matmul(q, np.swapaxes(k, -1, -2)) * scale
    if mask is not None:
        s = s + np.asarray(mask, dtype=np.float64)
    if is_causal:
        sq, skv = s.shape[-2], s.shape[-1]
        future = np.arange(skv)[None, :] > np.arange(sq)[:, None]
        s = np.where(future, -np.inf, s)
    m = np.max(s, axis=-1, keepdims=True)
    m = np.where(np.isfinite(m), m, 0.0)
    p = np.exp(s - m)
    l = p.sum(axis=-1, keepdims=True)
    linv = np.where(l > 1e-10, 1.0 / np.where(l > 1e-10, l, 1.0), 0.0)
    return np.matmul(p, v) * linv


def attention_rows(q, k, v, rows, scale=None, is_causal=False) -> np.ndarray:
    """Oracle for selected query rows of ONE (batch, head): q [Sq,D], k/v [Skv,D].
    Lets the full-size parity test sample rows without materialising S x S."""
    q = np.asarray(q, dtype=np.float64)
    k = np.asarray(k, dtype=np.float64)
    v = np.asarray(v, dtype=np.float64)
    rows = np.asarray(rows)
    d = q.shape[-1]
    if scale is None:
        scale = 1.0 / math.sqrt(d)
    s = (q[rows] @ k.T) * scale
    if is_causal:
        s = np.where(np.arange(k.shape[0])[None, :] > rows[:, None], -np.inf, s)
    m = s.max(axis=-1, keepdims=True)
    p = np.exp(s - m)
    return (p @ v) / p.sum(axis=-1, keepdims=True)


# --------------------------------------------------------------------------
# rotary position embedding and elementwise chains
# --------------------------------------------------------------------------
def rope(x, freqs) -> np.ndarray:
    """Compiler/CustomCallHandlers.swift:733-846: x [.., S, D] is split into halves x1 | x2 along the
    last axis; freqs is [S, D] with cos in the first half of a row and sin in the second (:783-808),
    or [S, D / 2] angles (:809-812); result [x1 cos - x2 sin | x1 sin + x2 cos]."""
    x = np.asarray(x, dtype=np.float64)
    f = np.asarray(freqs, dtype=np.float64)
    d = x.shape[-1]
    h = d // 2
    if d % 2 or x.ndim < 2:
        raise ValueError("x must be [.., S, D] with even D")
    f = f.reshape(-1, f.shape[-1])
    if f.shape[0] != x.shape[-2]:
        raise ValueError("freqs must have one row per position")
    if f.shape[1] == d:
        c, s = f[:, :h], f[:, h:]
    elif f.shape[1] == h:
        c, s = np.cos(f), np.sin(f)
    else:
        raise ValueError("freqs must be [S, D] or [S, D / 2]")
    x1, x2 = x[..., :h], x[..., h:]
    return np.concatenate([x1 * c - x2 * s, x1 * s + x2 * c], axis=-1)


def batch_norm(x, gamma, beta, mean, variance, eps: float = 1e-5) -> np.ndarray:
    """Compiler/CustomCallHandlers.swift:414-452 (`graph.normalize`): (x - mean) / sqrt(variance + eps) *
    gamma + beta with the four channel vectors spread along the last axis of x (the operands of the
    fusion pass, Compiler/PassManager.swift:1006-1080)."""
    x = np.asarray(x, dtype=np.float64)
    g, b, m, v = (np.asarray(t, dtype=np.float64).reshape(-1) for t in (gamma, beta, mean, variance))
    if not all(t.size == x.shape[-1] for t in (g, b, m, v)):
        raise ValueError("gamma, beta, mean and variance must have one element per channel")
    return (x - m) / np.sqrt(v + eps) * g + b


def depth_attention(q, k, v, scale: float = 1.0) -> np.ndarray:
    """Compiler/CustomCallHandlers.swift:1084-1140: softmax(q k^T scale, last axis) v for q [.., 1, H] or
    [.., H] and k, v [.., depth, H]; the result has q's shape."""
    q = np.asarray(q, dtype=np.float64)
    k = np.asarray(k, dtype=np.float64)
    v = np.asarray(v, dtype=np.float64)
    q3 = q.reshape(k.shape[:-2] + (1, k.shape[-1]))
    s = np.matmul(q3, np.swapaxes(k, -1, -2)) * scale
    s = s - s.max(axis=-1, keepdims=True)
    w = np.exp(s)
    w = w / w.sum(axis=-1, keepdims=True)
    return np.matmul(w, v).reshape(q.shape)


CHAIN_BINARY = {"add": np.add, "subtract": np.subtract, "multiply": np.multiply, "divide": np.divide,
                "maximum": np.maximum, "minimum": np.minimum}
CHAIN_UNARY = {"negate": np.negative, "abs": np.abs, "exponential": np.exp, "log": np.log, "sqrt": np.sqrt,
               "rsqrt": lambda v: 1.0 / np.sqrt(v), "tanh": np.tanh, "logistic": lambda v: 1.0 / (1.0 + np.exp(-v)),
               "sine": np.sin, "cosine": np.cos, "floor": np.floor, "ceil": np.ceil}


def elementwise_chain(inputs, ops) -> np.ndarray:
    """CustomCallHandlers.swift:927-1079: the running value starts as inputs[0]; a binary operation
    takes the next input as its right operand, a unary one transforms the running value."""
    if not ops:
        raise ValueError("No operations to fuse")
    cur = np.asarray(inputs[0], dtype=np.float64)
    k = 1
    for name in ops:
        if name in CHAIN_BINARY:
            if k >= len(inputs):
                raise ValueError(f"Not enough inputs for {name} operation")
            cur = CHAIN_BINARY[name](cur, np.asarray(inputs[k], dtype=np.float64))
            k += 1
        elif name in CHAIN_UNARY:
            cur = CHAIN_UNARY[name](cur)
        else:
            raise ValueError(f"Unsupported operation in fused chain: {name}")
    return cur


# --------------------------------------------------------------------------
# operator-level dispatch: custom_call target + JSON backend_config
# --------------------------------------------------------------------------
def custom_call(target: str, operands, backend_config: str = "") -> np.ndarray:
    """Evaluate one `stablehlo.custom_call @fused_*` the way the reference's
    handlers define it (Compiler/CustomCallHandlers.swift:75-89 for names,
    :102-168 for config parsing; an unparsable config is an empty dict)."""
    try:
        cfg = json.loads(backend_config) if backend_config else {}
        if not isinstance(cfg, dict):
            cfg = {}
    except ValueError:
        cfg = {}
    if target == "fused_scaled_dot_product_attention":
        if len(operands) < 3:
            raise ValueError("expected 3 inputs")
        q, k, v = operands[:3]
        scale = float(cfg.get("scale", 1.0))                      # :196
        has_mask = bool(cfg.get("has_mask", False))               # :197
        mask = operands[3] if (has_mask and len(operands) > 3) else None
        return attention(q, k, v, scale=scale,
                         is_causal=bool(cfg.get("is_causal", False)), mask=mask)
    if target == "fused_layer_norm":
        if len(operands) < 3:
            raise ValueError("expected 3 inputs")
        return layer_norm(operands[0], operands[1], operands[2], eps=float(cfg.get("eps", 1e-5)))
    if target == "fused_rms_norm":
        if len(operands) < 2:
            raise ValueError("expected 2 inputs")
        return rms_norm(operands[0], operands[1], eps=float(cfg.get("eps", 1e-5)))
    if target == "fused_softmax":
        return softmax(operands[0], axis=int(cfg.get("axis", -1)))
    if target == "fused_gelu":
        # tanh form whatever `approximate` says (CustomCallHandlers.swift:694-707); "erf": true is this
        # build's mark for a decomposed erf GELU and means the exact function
        return gelu_erf(operands[0]) if cfg.get("erf") is True else gelu_tanh(operands[0])
    if target == "fused_rope":
        if len(operands) < 2:
            raise ValueError("expected 2 inputs")
        return rope(operands[0], operands[1])
    if target == "fused_batch_norm":
        if len(operands) < 5:
            raise ValueError("expected 5 inputs")
        return batch_norm(*operands[:5], eps=float(cfg.get("eps", 1e-5)))            # CustomCallHandlers.swift:438
    if target == "fused_depth_attention":
        if len(operands) < 3:
            raise ValueError("expected 3 inputs")
        return depth_attention(*operands[:3], scale=float(cfg.get("scale", 1.0)))    # :1105
    if target == "fused_elementwise":
        ops = cfg.get("ops", cfg.get("operations"))               # CustomCallHandlers.swift:941-943
        if not isinstance(ops, list):
            raise ValueError("Missing 'ops' or 'operations' in fused_elementwise config")
        return elementwise_chain(operands, ops)
    if target == "fused_ffn":
        if len(operands) < 3:
            raise ValueError("expected 3 inputs")
        act = str(cfg.get("activation", "gelu"))                  # CustomCallHandlers.swift:870
        act = {"gelu_approximate": "gelu", "geluApproximate": "gelu", "swish": "silu"}.get(act, act)
        # an unknown name means no activation (CustomCallHandlers.swift:905); "is_gated" is ignored (:871)
        return gemm(ACTIVATIONS.get(act, ACTIVATIONS["none"])(gemm(operands[0], operands[1])), operands[2])
    if target == "fused_matmul_bias_activation":
        bias = operands[2] if len(operands) > 2 else None
        return matmul_bias_act(operands[0], operands[1], bias,
                               activation=str(cfg.get("activation", "none")),
                               trans_a=bool(cfg.get("trans_a", False)),
                               trans_b=bool(cfg.get("trans_b", False)))
    raise KeyError(target)


# --------------------------------------------------------------------------
# GPT-2 forward (composition; bf16 rounding points mirror the fused pipeline)
# --------------------------------------------------------------------------
def gpt2_forward(ids, params, n_head: int, compute_dtype: str = "bf16") -> np.ndarray:
    """Pre-LN GPT-2 forward with tied output head; returns float64 logits.

    Architecture constants from Sources/GPT2EndToEnd/main.swift:35-40. Each
    fused operator computes in wide precision from `compute_dtype`-rounded
    operands and rounds once at its output, which is the mixed-precision rule
    of the reference's 16-bit kernels (FlashAttentionKernel.swift:223-256,
    LayerNormKernel.swift:252-349).
    """
    r = lambda t: round_to(t, compute_dtype)
    ids = np.asarray(ids)
    bsz, seq = ids.shape
    wte, wpe = params["wte"], params["wpe"]
    d = wte.shape[1]
    hd = d // n_head
    wte = np.asarray(wte, np.float64)
    x = r(wte[ids] + np.asarray(wpe, np.float64)[None, :seq])
    for lyr in params["layers"]:
        h = r(layer_norm(x, r(lyr["ln1_g"]), r(lyr["ln1_b"]), 1e-5))
        qkv = r(gemm(h, r(lyr["w_qkv"])) + r(lyr["b_qkv"]))
        q, k, v = np.split(qkv, 3, axis=-1)
        sh = lambda t: t.reshape(bsz, seq, n_head, hd).transpose(0, 2, 1, 3)
        a = r(attention(sh(q), sh(k), sh(v), is_causal=True))
        a = a.transpose(0, 2, 1, 3).reshape(bsz, seq, d)
        x = r(x + r(gemm(a, r(lyr["w_o"])) + r(lyr["b_o"])))
        h = r(layer_norm(x, r(lyr["ln2_g"]), r(lyr["ln2_b"]), 1e-5))
        u = r(bias_gelu(gemm(h, r(lyr["w_fc"])), r(lyr["b_fc"])))
        x = r(x + r(gemm(u, r(lyr["w_proj"])) + r(lyr["b_proj"])))
    x = r(layer_norm(x, r(params["lnf_g"]), r(params["lnf_b"]), 1e-5))
    return gemm(x, r(wte).T)
