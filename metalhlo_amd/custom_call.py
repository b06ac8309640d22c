"""Operator-level entry: ``stablehlo.custom_call @fused_*`` with a JSON
``backend_config`` -> one gfx950 kernel launch.

Mirrors the reference's operator contract:

* target names and the registry — Compiler/CustomCallHandlers.swift:42-97
* config parsing (unparsable / empty config == {}), typed getters with
  defaults — BackendConfigParser, CustomCallHandlers.swift:102-168
* per-handler operand order, minimum operand counts and config keys —
  attention :179-278, layer norm :285-346, rms norm :353-394,
  matmul+bias+activation :456-560, softmax :644-672, gelu :677-711
* errors — CustomCallError.invalidInputCount / unsupportedTarget
"""
from __future__ import annotations

import json
import math
from typing import Any, Callable, Dict, List, Sequence

from . import kernels


class CustomCallError(RuntimeError):
    pass


class InvalidInputCount(CustomCallError):
    def __init__(self, expected: int, got: int):
        super().__init__(f"Invalid input count: expected {expected}, got {got}")
        self.expected, self.got = expected, got


class UnsupportedTarget(CustomCallError):
    pass


class BackendConfigParser:
    """CustomCallHandlers.swift:102-168."""

    @staticmethod
    def parse(config: str) -> Dict[str, Any]:
        if not config:
            return {}
        try:
            v = json.loads(config)
        except ValueError:
            return {}
        return v if isinstance(v, dict) else {}

    @staticmethod
    def get_float(cfg, key, default: float) -> float:
        v = cfg.get(key)
        if isinstance(v, bool) or not isinstance(v, (int, float)):
            return default
        return float(v)

    @staticmethod
    def get_int(cfg, key, default: int) -> int:
        v = cfg.get(key)
        if isinstance(v, bool) or not isinstance(v, (int, float)):
            return default
        return int(v)

    @staticmethod
    def get_bool(cfg, key, default: bool) -> bool:
        v = cfg.get(key)
        if isinstance(v, bool):
            return v
        if isinstance(v, int):
            return v != 0
        return default

    @staticmethod
    def get_string(cfg, key, default: str) -> str:
        v = cfg.get(key)
        return v if isinstance(v, str) else default

    @staticmethod
    def get_int_array(cfg, key, default: List[int]) -> List[int]:
        v = cfg.get(key)
        if isinstance(v, list) and all(isinstance(i, (int, float)) and not isinstance(i, bool) for i in v):
            return [int(i) for i in v]
        return default


P = BackendConfigParser


def _need(operands, n):
    if len(operands) < n:
        raise InvalidInputCount(n, len(operands))


def _last_axis_only(axes, rank, what):
    norm = sorted(a + rank if a < 0 else a for a in axes)
    if norm != [rank - 1]:
        raise CustomCallError(f"{what}: only normalisation over the last axis is supported, got axes {axes}")


def _sdpa(operands, cfg):
    _need(operands, 3)
    q, k, v = operands[:3]
    # handler default 1.0 (CustomCallHandlers.swift:196); the fusion passes always
    # write the scale explicitly (FusionPatterns.swift:689-731, PassManager.swift:633-638)
    scale = P.get_float(cfg, "scale", 1.0)
    has_mask = P.get_bool(cfg, "has_mask", False)
    mask = operands[3] if (has_mask and len(operands) > 3) else None
    is_causal = P.get_bool(cfg, "is_causal", False)
    return [kernels.flash_attention(q, k, v, scale=scale, is_causal=is_causal, mask=mask)]


def _layer_norm(operands, cfg):
    _need(operands, 3)
    x, gamma, beta = operands[:3]
    _last_axis_only(P.get_int_array(cfg, "axes", [-1]), x.dim(), "fused_layer_norm")
    return [kernels.layer_norm(x, gamma, beta, eps=P.get_float(cfg, "eps", 1e-5))]


def _rms_norm(operands, cfg):
    _need(operands, 2)
    x, w = operands[:2]
    _last_axis_only(P.get_int_array(cfg, "axes", [-1]), x.dim(), "fused_rms_norm")
    return [kernels.rms_norm(x, w, eps=P.get_float(cfg, "eps", 1e-5))]


def _softmax(operands, cfg):
    _need(operands, 1)
    return [kernels.softmax(operands[0], axis=P.get_int(cfg, "axis", -1))]


def _gelu(operands, cfg):
    _need(operands, 1)
    # the reference emits the tanh form whatever `approximate` says (:694-707); the pattern
    # recogniser of this build marks a decomposed erf GELU with "erf": true, which is exact
    return [kernels.gelu(operands[0], exact=P.get_bool(cfg, "erf", False))]


_ACTIVATION_ALIASES = {"gelu_approximate": "gelu", "geluApproximate": "gelu", "swish": "silu"}


def _ffn(operands, cfg):
    """act(x . up) . down, operands [x, up, down], config {activation: "gelu"}
    (CustomCallHandlers.swift:849-910).  As there, "is_gated" is read and ignored and an activation
    name the handler does not know means no activation; "gelu_exact" is the erf form here (the
    reference computes the tanh form for it)."""
    _need(operands, 3)
    x, up, down = operands[:3]
    act = P.get_string(cfg, "activation", "gelu")
    act = _ACTIVATION_ALIASES.get(act, act)
    if act not in kernels.ACTIVATION_CODE:
        act = "none"
    P.get_bool(cfg, "is_gated", False)          # reserved by the reference, ignored
    return [kernels.matmul(kernels.matmul(x, up, activation=act), down)]


def _rope(operands, cfg):
    """Rotary position embedding, operands [x, freqs] (CustomCallHandlers.swift:720-846)."""
    _need(operands, 2)
    return [kernels.rope(operands[0], operands[1])]


def _elementwise(operands, cfg):
    """A chain of elementwise operations, config {"ops": [...]} or {"operations": [...]}
    (CustomCallHandlers.swift:927-1079)."""
    ops = cfg.get("ops", cfg.get("operations"))
    if not isinstance(ops, list) or not all(isinstance(o, str) for o in ops):
        raise CustomCallError("Missing 'ops' or 'operations' in fused_elementwise config")
    _need(operands, 1)
    return [kernels.elementwise_chain(list(operands), ops)]


def _batch_norm(operands, cfg):
    """Normalisation with given statistics, operands [x, gamma, beta, mean, variance], config {eps}
    (CustomCallHandlers.swift:414-452)."""
    _need(operands, 5)
    x, gamma, beta, mean, var = operands[:5]
    return [kernels.batch_norm(x, gamma, beta, mean, var, eps=P.get_float(cfg, "eps", 1e-5))]


def _depth_attention(operands, cfg):
    """Attention of one query row over a few stored rows, operands [query, keys, values], config
    {scale} (CustomCallHandlers.swift:1084-1140)."""
    _need(operands, 3)
    q, k, v = operands[:3]
    return [kernels.depth_attention(q, k, v, scale=P.get_float(cfg, "scale", 1.0))]


def _matmul_bias_act(operands, cfg):
    _need(operands, 2)
    x, w = operands[:2]
    bias = operands[2] if len(operands) > 2 else None
    act = P.get_string(cfg, "activation", "none")
    act = _ACTIVATION_ALIASES.get(act, act)
    if act not in kernels.ACTIVATION_CODE:
        raise CustomCallError(f"fused_matmul_bias_activation: unknown activation '{act}'")
    return [kernels.matmul(x, w, bias=bias, activation=act,
                           trans_a=P.get_bool(cfg, "trans_a", False),
                           trans_b=P.get_bool(cfg, "trans_b", False))]


class CustomCallRegistry:
    """Compiler/CustomCallHandlers.swift:42-97."""

    def __init__(self):
        self._handlers: Dict[str, Callable] = {}
        for name, fn in (
            ("fused_scaled_dot_product_attention", _sdpa),
            ("fused_layer_norm", _layer_norm),
            ("fused_rms_norm", _rms_norm),
            ("fused_softmax", _softmax),
            ("fused_gelu", _gelu),
            ("fused_matmul_bias_activation", _matmul_bias_act),
            ("fused_ffn", _ffn),
            ("fused_rope", _rope),
            ("fused_elementwise", _elementwise),
            ("fused_batch_norm", _batch_norm),
            ("fused_depth_attention", _depth_attention),
        ):
            self.register(name, fn)

    def register(self, target: str, handler: Callable) -> None:
        self._handlers[target] = handler

    def has_handler(self, target: str) -> bool:
        return target in self._handlers

    @property
    def registered_targets(self) -> List[str]:
        return sorted(self._handlers)

    def emit(self, target: str, operands: Sequence, backend_config: str = ""):
        h = self._handlers.get(target)
        if h is None:
            raise UnsupportedTarget(f"Unsupported custom call target: {target}")
        return h(list(operands), BackendConfigParser.parse(backend_config))


shared = CustomCallRegistry()

# Targets the reference registers that lie outside the attention / GEMM / row-kernel
# path (CustomCallHandlers.swift:75-89); asking for them raises UnsupportedTarget.
NOT_ON_PATH = ("fused_conv_bias_act",)
