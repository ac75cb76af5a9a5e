"""SwiGLU feed-forward: d = (silu(x Wg^T) * (x Wu^T)) Wd^T without biases
(reference: Daisi.Llogos/Inference/ForwardPass.cs:240-246; silu Daisi.Llogos.Cpu/Silu.cs:9-16).
Gate and up are one stacked product whose row is [gate | up]."""
from __future__ import annotations

from typing import Callable, List, Optional

import torch

from .base import FeedForward, Residual, Runtime, StepContext, TensorSpec, mark, register_feed_forward
from .linear import Linear


@register_feed_forward("swiglu")
class SwiGLU(FeedForward):
    graph_safe = True
    takes_normed_rows = True
    adds_to_residual = True

    def __init__(self, prefix: str, hidden: int, intermediate: int):
        self.prefix = prefix
        self.hidden, self.intermediate = hidden, intermediate
        self.gate_up = Linear([prefix + "gate_proj", prefix + "up_proj"], hidden, [intermediate, intermediate], gated=True)
        self.down = Linear([prefix + "down_proj"], intermediate, [hidden])

    def tensor_specs(self) -> List[TensorSpec]:
        return self.gate_up.tensor_specs() + self.down.tensor_specs()

    def bind(self, get: Callable[[str], Optional[torch.Tensor]], rt: Runtime) -> None:
        super().bind(get, rt)
        self.gate_up.bind(get, rt)
        self.down.bind(get, rt)

    def forward(self, ctx: StepContext, h, residual: Optional[Residual] = None):
        act = self.gate_up.gated_product(h)
        if act is not None:
            # on packed weights silu(gate) * up is the epilogue of the gate/up product
            # (the reference's MatMulSwiGLU, Daisi.Llogos/IComputeBackend.cs:448-456)
            mark(ctx, "gate_up")
            out = self.down.add_to(act, residual) if residual is not None else None
            if out is None:
                out = self.down.product(act, f32_ok=True)
            mark(ctx, "down")
            return out
        gu = self.gate_up.product(h)
        mark(ctx, "gate_up")
        # otherwise silu(gate) * up is made inside the down product where its kernel can (few rows), by a
        # kernel of its own for many; the residual sum that follows adds the product's parts
        out = self.down.product(gu, swiglu_input=True, f32_ok=True)
        mark(ctx, "down")
        return out
