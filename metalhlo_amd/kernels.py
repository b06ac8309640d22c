"""Host-side launch helpers over the kernel C-ABI.

torch is used only as plumbing here: it owns device memory and the current HIP
stream.  Every function validates shapes, allocates the output and calls one
``mhip_*`` entry point through ctypes; none has a fallback implementation.

The names follow the reference's kernel registry
(Sources/MetalHLOCore/Metal/Kernels/KernelRegistry.swift:17): softmax,
layer_norm, rms_norm, gelu, flash_attention, plus matmul.
"""
from __future__ import annotations

import ctypes as C
import math
from typing import Optional

import torch

from . import _lib

# MHLOElementType numbering (Sources/CMetalHLO/include/metalhlo.h:62-76)
DTYPE_CODE = {
    torch.float16: 0, torch.float32: 1, torch.float64: 2, torch.bfloat16: 3, torch.bool: 4,
    torch.int8: 5, torch.int16: 6, torch.int32: 7, torch.int64: 8, torch.uint8: 9,
}
ACTIVATION_CODE = {"none": 0, "relu": 1, "gelu": 2, "silu": 3, "tanh": 4, "sigmoid": 5, "gelu_exact": 6}


def _code(t: torch.Tensor) -> int:
    try:
        return DTYPE_CODE[t.dtype]
    except KeyError:
        raise TypeError(f"unsupported dtype {t.dtype}") from None


def _dev(*ts):
    for t in ts:
        if t is None:
            continue
        if not t.is_cuda:
            raise RuntimeError("metalhlo_amd kernels need device tensors (no CPU path exists)")
        if not t.is_contiguous():
            raise ValueError("tensors must be dense row-major (contiguous)")


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


def softmax(x: torch.Tensor, axis: int = -1) -> torch.Tensor:
    _dev(x)
    lib = _lib.load()
    if axis < 0:
        axis += x.dim()
    if not 0 <= axis < x.dim():
        raise ValueError("softmax axis out of range")
    y = torch.empty_like(x)
    outer = math.prod(x.shape[:axis])
    inner = math.prod(x.shape[axis + 1:])
    n = x.shape[axis]
    if inner == 1:
        _lib.check(lib.mhip_softmax(_stream(), x.data_ptr(), y.data_ptr(), outer, n, _code(x)))
    else:
        _lib.check(lib.mhip_softmax_strided(_stream(), x.data_ptr(), y.data_ptr(), outer, n, inner,
                                            _code(x)))
    return y


def layer_norm(x, gamma=None, beta=None, eps: float = 1e-5):
    _dev(x, gamma, beta)
    lib = _lib.load()
    cols = x.shape[-1]
    for p in (gamma, beta):
        if p is not None and (p.numel() != cols or p.dtype != x.dtype):
            raise ValueError("gamma/beta must have the row length and dtype of x")
    y = torch.empty_like(x)
    _lib.check(lib.mhip_layer_norm(_stream(), x.data_ptr(), _ptr(gamma), _ptr(beta), y.data_ptr(),
                                   x.numel() // max(cols, 1), cols, eps, _code(x)))
    return y


def rms_norm(x, gamma=None, eps: float = 1e-5):
    _dev(x, gamma)
    lib = _lib.load()
    cols = x.shape[-1]
    if gamma is not None and (gamma.numel() != cols or gamma.dtype != x.dtype):
        raise ValueError("gamma must have the row length and dtype of x")
    y = torch.empty_like(x)
    _lib.check(lib.mhip_rms_norm(_stream(), x.data_ptr(), _ptr(gamma), y.data_ptr(),
                                 x.numel() // max(cols, 1), cols, eps, _code(x)))
    return y


def bias_gelu(x, bias=None, exact: bool = False):
    """gelu(x + bias): the tanh approximation, or with `exact` 0.5 v (1 + erf(v / sqrt 2))."""
    _dev(x, bias)
    lib = _lib.load()
    cols = x.shape[-1] if x.dim() else 1
    if bias is not None and (bias.numel() != cols or bias.dtype != x.dtype):
        raise ValueError("bias must have the row length and dtype of x")
    y = torch.empty_like(x)
    fn = lib.mhip_bias_gelu_erf if exact else lib.mhip_bias_gelu
    _lib.check(fn(_stream(), x.data_ptr(), _ptr(bias), y.data_ptr(), x.numel() // max(cols, 1), cols, _code(x)))
    return y


def gelu(x, exact: bool = False):
    return bias_gelu(x, None, exact)


def matmul(a, b, bias=None, activation: str = "none", trans_a: bool = False,
           trans_b: bool = False, out: Optional[torch.Tensor] = None,
           residual: Optional[torch.Tensor] = None):
    """act(op(a) @ op(b) + bias) (+ residual, which has the result's shape and may be `out`);
    leading dims of `a` are batch dims when `b` is batched too, otherwise they fold into M."""
    _dev(a, b, bias, out, residual)
    lib = _lib.load()
    if a.dtype != b.dtype:
        raise TypeError("operand dtypes differ")
    if b.dim() == 2:
        if trans_a and a.dim() != 2:
            raise ValueError("trans_a needs a 2-D lhs when rhs is 2-D")
        a2 = a if a.dim() == 2 else a.reshape(-1, a.shape[-1])
        batch, sa, sb = 1, 0, 0
        out_lead = tuple(a.shape[:-1]) if not trans_a else (a.shape[-1],)
    else:
        if a.dim() != b.dim() or a.shape[:-2] != b.shape[:-2]:
            raise ValueError("batched matmul needs equal batch dims")
        batch = math.prod(a.shape[:-2])
        a2 = a
        sa, sb = a.shape[-1] * a.shape[-2], b.shape[-1] * b.shape[-2]
        out_lead = tuple(a.shape[:-2]) + ((a.shape[-1],) if trans_a else (a.shape[-2],))
    M, K = (a2.shape[-1], a2.shape[-2]) if trans_a else (a2.shape[-2], a2.shape[-1])
    Kb, N = (b.shape[-1], b.shape[-2]) if trans_b else (b.shape[-2], b.shape[-1])
    if K != Kb:
        raise ValueError(f"contracting sizes differ: {K} vs {Kb}")
    if bias is not None and (bias.numel() != N or bias.dtype != a.dtype):
        raise ValueError("bias must be [N] of the operand dtype")
    if out is None:
        out = torch.empty(out_lead + (N,), dtype=a.dtype, device=a.device)
    if residual is None:
        _lib.check(lib.mhip_gemm(_stream(), a2.data_ptr(), b.data_ptr(), _ptr(bias), out.data_ptr(),
                                 M, N, K, batch, sa, sb, M * N, int(trans_a), int(trans_b),
                                 ACTIVATION_CODE[activation], _code(a)))
    else:
        if residual.numel() != out.numel() or residual.dtype != out.dtype:
            raise ValueError("residual must have the result's size and dtype")
        _lib.check(lib.mhip_gemm_residual(_stream(), a2.data_ptr(), b.data_ptr(), _ptr(bias), residual.data_ptr(),
                                          out.data_ptr(), M, N, K, batch, sa, sb, M * N, int(trans_a), int(trans_b),
                                          ACTIVATION_CODE[activation], _code(a)))
    return out


def flash_attention(q, k, v, scale: Optional[float] = None, is_causal: bool = False,
                    mask: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None):
    """softmax(scale * q k^T + mask, causal) v for [B,H,S,D] tensors.
    Default scale 1/sqrt(D) (FlashAttentionKernel.swift:55).  q, k, v (and `out`, when given)
    may be views with arbitrary batch / head / row strides as long as the last axis is
    contiguous, e.g. slices of a fused QKV projection; packed tensors take the plain entry."""
    for t in (q, k, v, out):
        if t is not None and (not t.is_cuda or t.dim() != 4 or t.stride(3) != 1):
            raise ValueError("attention operands must be 4-D device tensors with a contiguous last axis")
    _dev(mask)
    lib = _lib.load()
    if k.shape != v.shape or q.shape[:2] != k.shape[:2] or q.shape[3] != k.shape[3]:
        raise ValueError("expected q [B,H,Sq,D] and k,v [B,H,Skv,D]")
    if not (q.dtype == k.dtype == v.dtype):
        raise TypeError("q, k, v dtypes differ")
    B, H, Sq, D = q.shape
    Skv = k.shape[2]
    if scale is None:
        scale = 1.0 / math.sqrt(D)
    msb = msh = 0
    if mask is not None:
        if mask.dtype != q.dtype:
            raise TypeError("mask dtype must match q")
        while mask.dim() < 4:
            mask = mask.unsqueeze(0)
        if mask.shape[-2:] != (Sq, Skv) or mask.shape[0] not in (1, B) or mask.shape[1] not in (1, H):
            raise ValueError("mask must broadcast to [B,H,Sq,Skv] with full last two dims")
        msh = Sq * Skv if mask.shape[1] == H else 0
        msb = mask.shape[1] * Sq * Skv if mask.shape[0] == B else 0
    if out is None:
        out = torch.empty(q.shape, dtype=q.dtype, device=q.device)
    elif out.shape != q.shape or out.dtype != q.dtype:
        raise ValueError("out must have q's shape and dtype")
    if all(t.is_contiguous() for t in (q, k, v, out)):
        _lib.check(lib.mhip_flash_attention(_stream(), q.data_ptr(), k.data_ptr(), v.data_ptr(),
                                            _ptr(mask), out.data_ptr(), B, H, Sq, Skv, D, float(scale),
                                            int(is_causal), msb, msh, _code(q)))
    else:
        strides = (C.c_int64 * 12)(*[t.stride(i) for t in (q, k, v, out) for i in range(3)])
        _lib.check(lib.mhip_flash_attention_strided(_stream(), q.data_ptr(), k.data_ptr(), v.data_ptr(),
                                                    _ptr(mask), out.data_ptr(), B, H, Sq, Skv, D, float(scale),
                                                    int(is_causal), msb, msh, _code(q), C.addressof(strides)))
    return out


# ---- glue -------------------------------------------------------------------
def gather_rows(table, indices):
    _dev(table, indices)
    lib = _lib.load()
    row = math.prod(table.shape[1:])
    out = torch.empty(tuple(indices.shape) + tuple(table.shape[1:]), dtype=table.dtype,
                      device=table.device)
    _lib.check(lib.mhip_gather_rows(_stream(), table.data_ptr(), indices.data_ptr(), out.data_ptr(),
                                    indices.numel(), table.shape[0], row, _code(table),
                                    _code(indices)))
    return out


def embed_tokens(ids, wte, wpe, out_dtype):
    _dev(ids, wte, wpe)
    lib = _lib.load()
    if ids.dtype != torch.int32 or ids.dim() != 2:
        raise TypeError("ids must be int32 [B,S]")
    B, S = ids.shape
    if S > wpe.shape[0]:
        raise ValueError("sequence longer than the position table")
    out = torch.empty(B, S, wte.shape[1], dtype=out_dtype, device=ids.device)
    _lib.check(lib.mhip_embed_tokens(_stream(), ids.data_ptr(), wte.data_ptr(), wpe.data_ptr(),
                                     out.data_ptr(), B, S, wte.shape[1], wte.shape[0], _code(wte),
                                     DTYPE_CODE[out_dtype]))
    return out


def add(a, b):
    _dev(a, b)
    lib = _lib.load()
    if a.shape != b.shape or a.dtype != b.dtype:
        raise ValueError("add needs equal shapes and dtypes")
    y = torch.empty_like(a)
    _lib.check(lib.mhip_add(_stream(), a.data_ptr(), b.data_ptr(), y.data_ptr(), a.numel(), _code(a)))
    return y


def rope(x, freqs):
    """Rotary position embedding: x [.., S, D]; freqs [S, D] (cos | sin halves) or [S, D / 2] (angles)."""
    _dev(x, freqs)
    lib = _lib.load()
    if x.dim() < 2 or x.shape[-1] % 2 or freqs.dtype != x.dtype:
        raise ValueError("rope needs x [.., S, D] with even D and freqs of x's element type")
    S, D = x.shape[-2], x.shape[-1]
    fd = freqs.shape[-1] if freqs.dim() else 0
    if fd not in (D, D // 2) or freqs.numel() != S * fd:
        raise ValueError("rope: freqs must be [S, D] or [S, D / 2]")
    y = torch.empty_like(x)
    _lib.check(lib.mhip_rope(_stream(), x.data_ptr(), freqs.data_ptr(), y.data_ptr(), x.numel() // D if D else 0, S, D,
                             1 if fd == D // 2 else 0, _code(x)))
    return y


def batch_norm(x, gamma, beta, mean, variance, eps=1e-5):
    """y = (x - mean) / sqrt(variance + eps) * gamma + beta, the four vectors along x's last axis."""
    _dev(x, gamma, beta, mean, variance)
    lib = _lib.load()
    C_ = x.shape[-1] if x.dim() else 1
    for t in (gamma, beta, mean, variance):
        if t.numel() != C_ or t.dtype != x.dtype:
            raise ValueError("batch_norm: gamma, beta, mean and variance must be [channels] of x's element type")
    y = torch.empty_like(x)
    _lib.check(lib.mhip_batch_norm(_stream(), x.data_ptr(), gamma.data_ptr(), beta.data_ptr(), mean.data_ptr(), variance.data_ptr(),
                                   y.data_ptr(), x.numel() // C_ if C_ else 0, C_, float(eps), _code(x)))
    return y


def depth_attention(q, k, v, scale=1.0):
    """softmax(q k^T scale) v for one query row per leading index: q [.., 1, H] or [.., H], k and v
    [.., depth, H] with depth <= 64; the result has q's shape."""
    _dev(q, k, v)
    lib = _lib.load()
    if k.dim() < 2 or k.shape != v.shape or not (q.dtype == k.dtype == v.dtype):
        raise ValueError("depth_attention: k and v must be [.., depth, H] of q's element type")
    depth, H = k.shape[-2], k.shape[-1]
    lead = tuple(k.shape[:-2])
    if tuple(q.shape) not in (lead + (1, H), lead + (H,)):
        raise ValueError("depth_attention: q must be [.., 1, H] or [.., H] over k's leading axes")
    out = torch.empty_like(q)
    rows = q.numel() // H if H else 0
    _lib.check(lib.mhip_depth_attention(_stream(), q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), rows, depth, H,
                                        float(scale), _code(q)))
    return out


CHAIN_UNARY_CODE = {"exponential": 0, "tanh": 1, "rsqrt": 2, "sqrt": 3, "negate": 4, "logistic": 5, "abs": 6, "log": 7,
                    "sine": 9, "cosine": 10, "floor": 11, "ceil": 12}
CHAIN_BINARY_CODE = {"add": 100, "subtract": 101, "multiply": 102, "divide": 103, "maximum": 104, "minimum": 105}


def elementwise_chain(inputs, ops):
    """One launch for a chain of elementwise operations: the running value starts as inputs[0], a
    binary operation takes the next input as its right operand, a unary one transforms the running
    value.  Inputs have the result's shape (that of inputs[0]) or one element."""
    import ctypes as C
    _dev(*inputs)
    lib = _lib.load()
    codes = []
    for name in ops:
        if name in CHAIN_BINARY_CODE:
            codes.append(CHAIN_BINARY_CODE[name])
        elif name in CHAIN_UNARY_CODE:
            codes.append(CHAIN_UNARY_CODE[name])
        else:
            raise ValueError(f"Unsupported operation in fused chain: {name}")
    need = 1 + sum(c >= 100 for c in codes)
    if len(inputs) < need:
        raise ValueError("Not enough inputs for the operations of the chain")
    inputs = list(inputs[:need])
    if any(t.dtype != inputs[0].dtype for t in inputs):
        raise ValueError("every input must have one element type")
    shape = max((t.shape for t in inputs), key=lambda sh: int(torch.Size(sh).numel()))
    y = torch.empty(shape, dtype=inputs[0].dtype, device=inputs[0].device)
    ptrs = (C.c_void_p * need)(*[t.data_ptr() for t in inputs])
    counts = (C.c_int64 * need)(*[t.numel() for t in inputs])
    arr = (C.c_int32 * len(codes))(*codes)
    _lib.check(lib.mhip_elementwise_chain(_stream(), need, ptrs, counts, len(codes), arr, y.data_ptr(), y.numel(), _code(y)))
    return y


def convert(x, dtype):
    _dev(x)
    lib = _lib.load()
    y = torch.empty(x.shape, dtype=dtype, device=x.device)
    _lib.check(lib.mhip_convert(_stream(), x.data_ptr(), y.data_ptr(), x.numel(), _code(x),
                                DTYPE_CODE[dtype]))
    return y


def transpose_0213(x):
    _dev(x)
    lib = _lib.load()
    d0, d1, d2, d3 = x.shape
    y = torch.empty(d0, d2, d1, d3, dtype=x.dtype, device=x.device)
    _lib.check(lib.mhip_transpose_0213(_stream(), x.data_ptr(), y.data_ptr(), d0, d1, d2, d3,
                                       _code(x)))
    return y


def split_qkv_heads(qkv, n_head: int):
    _dev(qkv)
    lib = _lib.load()
    B, S, three_d = qkv.shape
    D = three_d // (3 * n_head)
    q, k, v = (torch.empty(B, n_head, S, D, dtype=qkv.dtype, device=qkv.device) for _ in range(3))
    _lib.check(lib.mhip_split_qkv_heads(_stream(), qkv.data_ptr(), q.data_ptr(), k.data_ptr(),
                                        v.data_ptr(), B, S, n_head, D, _code(qkv)))
    return q, k, v


def iota(shape, dim: int, dtype, device="cuda"):
    lib = _lib.load()
    y = torch.empty(shape, dtype=dtype, device=device)
    _lib.check(lib.mhip_iota(_stream(), y.data_ptr(), math.prod(shape[:dim]), shape[dim],
                             math.prod(shape[dim + 1:]), DTYPE_CODE[dtype]))
    return y


def argmax(x, index_dtype=torch.int32, return_values: bool = False):
    _dev(x)
    lib = _lib.load()
    cols = x.shape[-1]
    idx = torch.empty(x.shape[:-1], dtype=index_dtype, device=x.device)
    val = torch.empty(x.shape[:-1], dtype=x.dtype, device=x.device) if return_values else None
    _lib.check(lib.mhip_argmax(_stream(), x.data_ptr(), idx.data_ptr(), _ptr(val),
                               x.numel() // cols, cols, _code(x), DTYPE_CODE[index_dtype]))
    return (idx, val) if return_values else idx


def autotune_matmul(a, b, bias=None, activation: str = "none", trans_a: bool = False,
                    trans_b: bool = False, iters: int = 10):
    """Times the GEMM kernel variants for this 2-D problem and stores the fastest in the
    library's tuning table (used by every later matmul of the same shape, layout and
    type).  Returns (variant code 128 | 256 | 2560 | 2561, microseconds per launch)."""
    _dev(a, b, bias)
    lib = _lib.load()
    if a.dim() != 2 or b.dim() != 2 or a.dtype != b.dtype:
        raise ValueError("autotune_matmul takes two 2-D operands of one dtype")
    M, K = (a.shape[1], a.shape[0]) if trans_a else (a.shape[0], a.shape[1])
    N = b.shape[0] if trans_b else b.shape[1]
    out = torch.empty((M, N), dtype=a.dtype, device=a.device)
    variant, us = C.c_int(0), C.c_float(0.0)
    _lib.check(lib.mhip_gemm_autotune(_stream(), a.data_ptr(), b.data_ptr(), _ptr(bias), out.data_ptr(), M, N, K, 1,
                                      0, 0, M * N, int(trans_a), int(trans_b), ACTIVATION_CODE[activation], _code(a),
                                      int(iters), C.byref(variant), C.byref(us)))
    return variant.value, us.value


def autotune_row(op: str, x, gamma=None, beta=None, eps: float = 1e-5, iters: int = 10):
    """Times the launch forms of a row operator ("softmax", "layer_norm", "rms_norm") for x
    [rows, cols] and stores the fastest in the tuning table.  Returns ((kind, rows per wave
    group, ordered, workgroups per CU), microseconds per launch)."""
    _dev(x, gamma, beta)
    lib = _lib.load()
    code = {"softmax": 0, "layer_norm": 1, "rms_norm": 2}[op]
    cols = x.shape[-1]
    out = torch.empty_like(x)
    choice, us = (C.c_int * 4)(), C.c_float(0.0)
    _lib.check(lib.mhip_row_autotune(_stream(), code, x.data_ptr(), _ptr(gamma), _ptr(beta), out.data_ptr(),
                                     x.numel() // cols, cols, float(eps), _code(x), int(iters), choice, C.byref(us)))
    return tuple(choice), us.value


def autotune_attention(q, k, v, scale=None, is_causal: bool = False, iters: int = 5):
    """Times the attention kernels that can serve packed q [B,H,Sq,D], k, v [B,H,Skv,D] and stores
    the fastest in the tuning table.  Returns (variant 1 | 2 | 3, microseconds per launch)."""
    _dev(q, k, v)
    lib = _lib.load()
    B, H, Sq, D = q.shape
    out = torch.empty_like(q)
    variant, us = C.c_int(0), C.c_float(0.0)
    _lib.check(lib.mhip_attention_autotune(_stream(), q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), B, H, Sq,
                                           k.shape[2], D, float(D ** -0.5 if scale is None else scale), int(is_causal),
                                           _code(q), int(iters), C.byref(variant), C.byref(us)))
    return variant.value, us.value


def tuning_device() -> str:
    """The current device's key in the tuning table (architecture name / compute units)."""
    return _lib.load().mhip_tuning_device().decode()


def tuning_save(path: str) -> None:
    _lib.check(_lib.load().mhip_tuning_save(str(path).encode()))


def tuning_load(path: str) -> None:
    _lib.check(_lib.load().mhip_tuning_load(str(path).encode()))


def shipped_tuning_table() -> str:
    """Path of the table that ships for the current device (it may not exist); the kernel library
    loads it by itself at first use unless the table was cleared before."""
    import os
    return os.path.join(os.path.dirname(os.path.abspath(__file__)), "tuning", tuning_device().replace("/", "_") + ".txt")


def tuning_clear() -> None:
    _lib.load().mhip_tuning_clear()


def tuning_count() -> int:
    return _lib.load().mhip_tuning_count()
