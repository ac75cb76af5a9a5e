"""Grouped-query attention over the paged cache.

Order inside the mixer (reference: Daisi.Llogos/Inference/ForwardPass.cs:329-405):
projections q, k, v (:368-370) with their optional biases (:379-382; a bias is part of its
projection here), optional per-head RMSNorm of q and k with one weight per projection
(:372-376), rotation (:385), cache write (:388), attention with kv head = head / group and
scale 1/sqrt(head_dim) after the dot (:336, :391-401), output projection (:404).
"""
from __future__ import annotations

import math
from typing import Callable, List, Optional

import torch

from ..ops import kernels as K
from .base import KVSpec, LayerCache, Mixer, Residual, Runtime, StepContext, TensorSpec, mark, register_mixer
from .linear import Linear
from .rope import Rotary


@register_mixer("attention")
class Attention(Mixer):
    graph_safe = True
    takes_normed_rows = True       # h goes into the q/k/v product alone
    adds_to_residual = True        # the output projection can add itself to the stream

    def __init__(self, prefix: str, hidden: int, n_heads: int, n_kv_heads: int, head_dim: int,
                 position: Rotary, bias: bool = False, qk_norm: bool = False, eps: float = 1e-6,
                 window: int = 0, sinks: int = 0, scale: Optional[float] = None):
        if n_heads % n_kv_heads:
            raise ValueError(f"{n_heads} heads are not a multiple of {n_kv_heads} kv heads")
        if head_dim % 16 or head_dim > K.MAX_HEAD_DIM:
            raise ValueError(f"head_dim {head_dim} must be a multiple of 16, at most {K.MAX_HEAD_DIM}")
        self.prefix = prefix
        self.hidden = hidden
        self.n_heads, self.n_kv_heads, self.head_dim = n_heads, n_kv_heads, head_dim
        self.position = position
        self.qk_norm = qk_norm
        self.eps = float(eps)
        self.window, self.sinks = int(window), int(sinks)
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(head_dim)
        q_w, kv_w = n_heads * head_dim, n_kv_heads * head_dim
        self.qkv = Linear([prefix + "q_proj", prefix + "k_proj", prefix + "v_proj"], hidden,
                          [q_w, kv_w, kv_w], bias=bias)
        self.o = Linear([prefix + "o_proj"], q_w, [hidden])
        self.q_norm_w: Optional[torch.Tensor] = None
        self.k_norm_w: Optional[torch.Tensor] = None
        self.fuse_decode = True     # single-token steps: one kernel from the projection to the attention output

    def kv_spec(self) -> KVSpec:
        return KVSpec(self.n_kv_heads, self.head_dim, self.window, self.sinks)

    def tensor_specs(self) -> List[TensorSpec]:
        specs = self.qkv.tensor_specs() + self.o.tensor_specs()
        if self.qk_norm:
            specs.append(TensorSpec(self.prefix + "q_norm.weight", (self.head_dim,), "norm"))
            specs.append(TensorSpec(self.prefix + "k_norm.weight", (self.head_dim,), "norm"))
        return specs

    def bind(self, get: Callable[[str], Optional[torch.Tensor]], rt: Runtime) -> None:
        super().bind(get, rt)
        self.qkv.bind(get, rt)
        self.o.bind(get, rt)
        if self.qk_norm:
            self.q_norm_w = get(self.prefix + "q_norm.weight").to(device=rt.device, dtype=torch.float32).contiguous()
            self.k_norm_w = get(self.prefix + "k_norm.weight").to(device=rt.device, dtype=torch.float32).contiguous()
        if getattr(self.position, "inv_freq", None) is None:
            self.position.bind(get, rt)

    def forward(self, ctx: StepContext, h, cache: LayerCache, residual: Optional[Residual] = None):
        nh, nkv, hd = self.n_heads, self.n_kv_heads, self.head_dim
        cs = self.position.prepare(ctx)
        if cache.writes:
            qkv = self.qkv.product(h, f32_ok=True)                      # [(parts,) T, (nh + 2 nkv) hd]
            mark(ctx, "qkv")
            if ctx.is_decode and self.fuse_decode:
                # one token a sequence: norm, rotation and cache write inside the attention kernel
                a = K.attention_decode_fused(ctx, qkv, self.qkv.bias_rows(), nh, nkv, hd, self.position.rot,
                                             self.position.pairing, self.q_norm_w, self.k_norm_w, self.eps, cs,
                                             cache.k_pool, cache.v_pool, cache.table, self.scale, self.window,
                                             self.sinks)
                if a is not None:
                    mark(ctx, "attention")
                    return self._project(ctx, a, residual)
            q = K.qk_rope_cache(qkv, self.qkv.bias_rows(), self.rt.dtype, nh, nkv, hd, self.position.rot,
                                self.position.pairing, self.q_norm_w, self.k_norm_w, self.eps, cs,
                                cache.k_pool, cache.v_pool, cache.table, ctx.tok_seq, ctx.tok_pos)
        else:
            # the keys and values of these positions are another layer's: project q alone
            qkv = self.qkv.product(h, rows_out=nh * hd, f32_ok=True)
            mark(ctx, "qkv")
            q = K.qk_rope_cache(qkv, self.qkv.bias_rows(nh * hd), self.rt.dtype, nh, 0, hd, self.position.rot,
                                self.position.pairing, self.q_norm_w, None, self.eps, cs, None, None, None,
                                ctx.tok_seq, ctx.tok_pos)
        mark(ctx, "rotation")
        a = K.attention(ctx, q, q.stride(0), cache.k_pool, cache.v_pool, cache.table,
                        nh, nkv, hd, self.scale, self.window, self.sinks)
        mark(ctx, "attention")
        return self._project(ctx, a, residual)

    def _project(self, ctx: StepContext, a: torch.Tensor, residual: Optional[Residual] = None):
        out = self.o.add_to(a, residual) if residual is not None else None
        if out is None:
            out = self.o.product(a, f32_ok=True)    # the residual sum that follows adds the parts
        mark(ctx, "o")
        return out
