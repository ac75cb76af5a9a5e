"""Arrangement of a layer's parts.  The pre-norm residual block:

    x += pending;  a = mixer(norm1(x));  x += a;  d = ffn(norm2(x));  pending = d

Each residual sum is done inside the following norm's kernel, in float32, so the
feed-forward's output is handed on as `pending` and added by whoever norms next
(reference: the deferred adds of Daisi.Llogos/Inference/ForwardPass.cs:214-252)."""
from __future__ import annotations

from typing import Callable, List, Optional, Tuple

import torch

from .base import Block, FeedForward, LayerCache, Mixer, Norm, Part, Runtime, StepContext, TensorSpec, mark, register_block


@register_block("pre_norm")
class PreNormBlock(Block):
    def __init__(self, mixer_norm: Norm, mixer: Mixer, ffn_norm: Norm, ffn: FeedForward):
        self.mixer_norm, self.mixer, self.ffn_norm, self.ffn = mixer_norm, mixer, ffn_norm, ffn

    def mixers(self) -> List[Mixer]:
        return [self.mixer]

    def feed_forwards(self) -> List[FeedForward]:
        return [self.ffn]

    def parts(self) -> List[Part]:
        return [self.mixer_norm, self.mixer, self.ffn_norm, self.ffn]

    def forward(self, ctx: StepContext, x: torch.Tensor, pending: Optional[torch.Tensor],
                caches) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
        cache = caches[0] if isinstance(caches, (list, tuple)) else caches
        h = self.mixer_norm.forward(x, pending)
        mark(ctx, "norm")
        a = self.mixer.forward(ctx, h, cache)
        mark(ctx, "mixer")
        h = self.ffn_norm.forward(x, a)
        mark(ctx, "norm")
        d = self.ffn.forward(ctx, h)
        mark(ctx, "feed_forward")
        return x, d
