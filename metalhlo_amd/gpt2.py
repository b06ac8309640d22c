"""GPT-2 forward through the fused kernels (the GPT-2-small benchmark configuration: B8 S1024).

The op sequence is the one the reference's fusion passes produce for a pre-LN
GPT-2 block — fused_layer_norm, fused_matmul_bias_activation (bias only, and
bias + tanh-GELU), fused_scaled_dot_product_attention with is_causal, residual
adds, token + position gather, tied output head — issued in order on one HIP
stream like the reference's integrated executor does
(Sources/MetalHLOCore/Runtime/IntegratedExecutor.swift:208-232), but with no
host synchronisation between launches.  Architecture constants:
Sources/GPT2EndToEnd/main.swift:35-40.

Parameters are held in fp32; every forward converts them to the compute type at
use (the `convert` ops of the fp32-params / bf16-compute graph), computes each
fused op with fp32 accumulation and rounds once at its output.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List

import numpy as np
import torch

from . import kernels


@dataclass
class GPT2Config:
    n_layer: int = 12
    d_model: int = 768
    n_head: int = 12
    d_ff: int = 3072
    vocab: int = 50257
    n_pos: int = 1024


def init_params(cfg: GPT2Config, seed: int = 5) -> Dict:
    """Random-init N(0, 0.02) weights, zero biases, LN gamma 1 / beta 0 (numpy fp32)."""
    rng = np.random.default_rng(seed)
    d, f = cfg.d_model, cfg.d_ff
    w = lambda *s: rng.normal(0.0, 0.02, s).astype(np.float32)
    z = lambda *s: np.zeros(s, np.float32)
    o = lambda *s: np.ones(s, np.float32)
    layers = [dict(ln1_g=o(d), ln1_b=z(d), w_qkv=w(d, 3 * d), b_qkv=z(3 * d), w_o=w(d, d), b_o=z(d),
                   ln2_g=o(d), ln2_b=z(d), w_fc=w(d, f), b_fc=z(f), w_proj=w(f, d), b_proj=z(d))
              for _ in range(cfg.n_layer)]
    return dict(wte=w(cfg.vocab, d), wpe=w(cfg.n_pos, d), layers=layers, lnf_g=o(d), lnf_b=z(d))


class GPT2:
    def __init__(self, cfg: GPT2Config, params: Dict, compute_dtype=torch.bfloat16, device="cuda"):
        self.cfg, self.dtype = cfg, compute_dtype
        # All parameters live in ONE fp32 device buffer (each tensor starts on a
        # 16-byte boundary), so the per-step fp32 -> compute-type conversion is a
        # single streaming launch; the named entries are views into the buffers.
        flat, self._slots = [], []

        def put(path, a):
            a = np.ascontiguousarray(a, dtype=np.float32)
            off = sum(x.size for x in flat)
            pad = (-a.size) % 8
            flat.append(np.concatenate([a.reshape(-1), np.zeros(pad, np.float32)]))
            self._slots.append((path, off, a.shape))

        # the tied output head multiplies by wte^T: rows padded with zeros to a multiple of 64
        # keep that GEMM on the aligned kernels; "wte" is the view of the real rows
        wte = np.asarray(params["wte"], dtype=np.float32)
        self.vocab_pad = -(-wte.shape[0] // 64) * 64
        put(("wte_pad",), np.concatenate([wte, np.zeros((self.vocab_pad - wte.shape[0], wte.shape[1]), np.float32)]))
        self._slots.append((("wte",), self._slots[-1][1], wte.shape))
        for name in ("wpe", "lnf_g", "lnf_b"):
            put((name,), params[name])
        for i, l in enumerate(params["layers"]):
            for k, v in l.items():
                put(("layers", i, k), v)
        self.flat32 = torch.from_numpy(np.concatenate(flat)).to(device)
        self.p32 = self._views(self.flat32)

    def _views(self, flat: torch.Tensor) -> Dict:
        out: Dict = {"layers": [dict() for _ in range(self.cfg.n_layer)]}
        for path, off, shape in self._slots:
            v = flat[off:off + int(np.prod(shape))].view(*shape)
            if path[0] == "layers":
                out["layers"][path[1]][path[2]] = v
            else:
                out[path[0]] = v
        return out

    def forward(self, ids: torch.Tensor) -> torch.Tensor:
        """ids int32 [B,S] on the device -> logits [B,S,vocab] in the compute type."""
        cfg = self.cfg
        B, S = ids.shape
        d, H = cfg.d_model, cfg.n_head
        # the graph's `convert` ops: fp32 parameters -> compute type, every step
        p = self.p32 if self.dtype == torch.float32 else self._views(kernels.convert(self.flat32, self.dtype))
        x = kernels.embed_tokens(ids, self.p32["wte"], self.p32["wpe"], self.dtype).reshape(B * S, d)
        # the strided attention entry covers 16-bit types and head sizes 64 / 128
        in_place = self.dtype in (torch.bfloat16, torch.float16) and d // H in (64, 128)
        for l in p["layers"]:
            h = kernels.layer_norm(x, l["ln1_g"], l["ln1_b"], eps=1e-5)
            qkv = kernels.matmul(h, l["w_qkv"], bias=l["b_qkv"])
            if in_place:
                # attention reads Q, K, V in place ([B,S,3,H,D] views of the projection) and
                # writes [B,S,H,D]: no head split / merge passes over memory
                q, k, v = qkv.view(B, S, 3, H, d // H).permute(2, 0, 3, 1, 4).unbind(0)
                a = torch.empty(B, S, H, d // H, dtype=qkv.dtype, device=qkv.device)
                kernels.flash_attention(q, k, v, is_causal=True, out=a.permute(0, 2, 1, 3))
                a = a.view(B * S, d)
            else:
                q, k, v = kernels.split_qkv_heads(qkv.reshape(B, S, 3 * d), H)
                a = kernels.flash_attention(q, k, v, is_causal=True)
                a = kernels.transpose_0213(a).reshape(B * S, d)
            x = kernels.matmul(a, l["w_o"], bias=l["b_o"], residual=x)          # x + proj(a), one kernel
            h = kernels.layer_norm(x, l["ln2_g"], l["ln2_b"], eps=1e-5)
            u = kernels.matmul(h, l["w_fc"], bias=l["b_fc"], activation="gelu")
            x = kernels.matmul(u, l["w_proj"], bias=l["b_proj"], residual=x)
        x = kernels.layer_norm(x, p["lnf_g"], p["lnf_b"], eps=1e-5)
        logits = kernels.matmul(x, p["wte_pad"], trans_b=True)   # tied head: x . wte^T (padded columns are 0)
        return logits.reshape(B, S, self.vocab_pad)[..., :cfg.vocab]

    def capture(self, ids: torch.Tensor) -> "GraphedForward":
        """Records one forward pass for ids of this shape into a HIP graph.  Every launch
        of the pass goes to the stream handed to the kernel library, so the whole
        pipeline (about 135 launches) replays with one submission instead of one host
        call per kernel."""
        static_ids = ids.clone()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):           # first calls set kernel attributes; keep them out of the capture
            for _ in range(2):
                self.forward(static_ids)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            logits = self.forward(static_ids)
        return GraphedForward(graph, static_ids, logits)

    @staticmethod
    def flops(cfg: GPT2Config, B: int, S: int) -> float:
        d, f = cfg.d_model, cfg.d_ff
        per_tok = cfg.n_layer * (d * 3 * d + d * d + 2 * d * f) + d * cfg.vocab
        attn = cfg.n_layer * 2 * B * cfg.n_head * S * S * (d // cfg.n_head)   # causal: half of 4BHS^2D
        return 2.0 * per_tok * B * S + attn


class GraphedForward:
    """A captured forward pass: copy new token ids in, replay, read `logits` (a buffer
    owned by the graph, overwritten by the next replay)."""

    def __init__(self, graph, ids: torch.Tensor, logits: torch.Tensor):
        self.graph, self.ids, self.logits = graph, ids, logits

    def __call__(self, ids: torch.Tensor) -> torch.Tensor:
        if ids.shape != self.ids.shape or ids.dtype != self.ids.dtype:
            raise ValueError("captured for ids of shape %s" % (tuple(self.ids.shape),))
        self.ids.copy_(ids)
        self.graph.replay()
        return self.logits
