"""RMSNorm with the residual sum fused in.
out = v * rsqrt(mean(v^2) + eps) * w with v = x + delta; eps inside the root and the weight
as it is (reference: Daisi.Llogos.Cpu/RmsNorm.cs:14-65; fused forms
Daisi.Llogos/IComputeBackend.cs:417-466)."""
from __future__ import annotations

from typing import Callable, List, Optional

import torch

from ..ops import kernels as K
from .base import Norm, NormedRows, Runtime, TensorSpec, register_norm


@register_norm("rmsnorm")
class RMSNorm(Norm):
    takes_row_squares = True

    def __init__(self, name: str, width: int, eps: float):
        self.name = name
        self.width = width
        self.eps = float(eps)
        self.weight: Optional[torch.Tensor] = None

    def tensor_specs(self) -> List[TensorSpec]:
        return [TensorSpec(self.name + ".weight", (self.width,), "norm")]

    def bind(self, get: Callable[[str], Optional[torch.Tensor]], rt: Runtime) -> None:
        super().bind(get, rt)
        self.weight = get(self.name + ".weight").to(device=rt.device, dtype=torch.float32).contiguous()

    def forward(self, x: torch.Tensor, delta=None, rows: Optional[torch.Tensor] = None,
                write_back: bool = True, lazy: bool = False):
        if isinstance(delta, K.RowSquares):
            # the product before has added itself to x; if it also left this norm's rows without their
            # scale, a consumer that takes them needs no kernel here
            if lazy and rows is None and delta.unscaled is not None and delta.norm_w is self.weight:
                return NormedRows(delta, self.eps, self, x)
            delta = None
        return K.rmsnorm(x, self.weight, self.eps, self.rt.dtype, delta=delta, rows=rows, write_back=write_back)

    def row_weight(self) -> Optional[torch.Tensor]:
        return self.weight
