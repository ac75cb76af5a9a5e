"""Arrangement of a layer's parts.  The pre-norm residual block:

    x += pending;  a = mixer(norm1(x));  x += a;  d = ffn(norm2(x));  pending = d

Each residual sum is done inside the following norm's kernel, in float32, so the
feed-forward's output is handed on as `pending` and added by whoever norms next
(reference: the deferred adds of Daisi.Llogos/Inference/ForwardPass.cs:214-252); or, for
steps of few rows, by the product that closes the mixer or the feed-forward, which then also
leaves the following norm's rows for the product that opens the next part."""
from __future__ import annotations

from typing import Callable, List, Optional, Tuple

import torch

from .base import Block, FeedForward, LayerCache, Mixer, Norm, Part, Residual, Runtime, StepContext, TensorSpec, mark, register_block


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

    takes_next_norm = True

    def entry_norm(self) -> Optional[Norm]:
        return self.mixer_norm

    @staticmethod
    def _norm(norm: Norm, x: torch.Tensor, delta, lazy: bool):
        # (only a norm that knows of unscaled rows is asked for them)
        return norm.forward(x, delta, lazy=True) if lazy and norm.takes_row_squares else norm.forward(x, delta)

    def forward(self, ctx: StepContext, x: torch.Tensor, pending, caches, next_norm: Optional[Norm] = None):
        cache = caches[0] if isinstance(caches, (list, tuple)) else caches
        # A part that says so may add its output to x itself and leave the next norm's rows half made
        # (then `a` or `d` is what it left, and the norm that takes it needs no kernel of its own).
        h = self._norm(self.mixer_norm, x, pending, self.mixer.takes_normed_rows)
        mark(ctx, "norm")
        if self.mixer.adds_to_residual and self.ffn_norm.takes_row_squares:
            a = self.mixer.forward(ctx, h, cache, residual=Residual(x, self.ffn_norm))
        else:
            a = self.mixer.forward(ctx, h, cache)
        mark(ctx, "mixer")
        h = self._norm(self.ffn_norm, x, a, self.ffn.takes_normed_rows)
        mark(ctx, "norm")
        if self.ffn.adds_to_residual and next_norm is not None and next_norm.takes_row_squares:
            d = self.ffn.forward(ctx, h, residual=Residual(x, next_norm))
        else:
            d = self.ffn.forward(ctx, h)
        mark(ctx, "feed_forward")
        return x, d
