"""Rotary position encoding: base, rotated width, pairing and frequency scaling are
parameters.  f_i = theta^(-2i/rot) in double (reference: Daisi.Llogos.Cpu/Rope.cs:145-162);
a scaling rule divides each f_i by a per-pair factor, the reference's mechanism for
frequency factors (Rope.cs:42-63).  The Llama-3 rule fills that table from the
configuration: short wavelengths keep their frequency, long ones are slowed by `factor`,
the band between is interpolated."""
from __future__ import annotations

import math
from typing import Callable, List, Optional

import torch

from ..ops import kernels as K
from .base import PositionEncoding, Runtime, StepContext, register_position

SPLIT_HALF, INTERLEAVED = 0, 1


def inverse_frequencies(rot: int, theta: float) -> List[float]:
    return [1.0 / math.pow(float(theta), 2.0 * i / rot) for i in range(rot // 2)]


def llama3_factors(freqs: List[float], factor: float, low_freq_factor: float, high_freq_factor: float,
                   original_max_position: int) -> List[float]:
    low_wavelen = original_max_position / low_freq_factor
    high_wavelen = original_max_position / high_freq_factor
    out = []
    for f in freqs:
        wavelen = 2.0 * math.pi / f
        if wavelen < high_wavelen:
            out.append(1.0)
        elif wavelen > low_wavelen:
            out.append(float(factor))
        else:
            smooth = (original_max_position / wavelen - low_freq_factor) / (high_freq_factor - low_freq_factor)
            out.append(1.0 / ((1.0 - smooth) / factor + smooth))
    return out


@register_position("rotary")
class Rotary(PositionEncoding):
    def __init__(self, head_dim: int, rot: int, theta: float, pairing: str = "split_half",
                 scaling: Optional[dict] = None):
        if rot <= 0 or rot % 2 or rot > head_dim:
            raise ValueError(f"rotary width {rot} must be even and within head_dim {head_dim}")
        if pairing not in ("split_half", "interleaved"):
            raise ValueError(f"unknown rotary pairing '{pairing}'")
        self.head_dim = head_dim
        self.rot = rot
        self.theta = float(theta)
        self.pairing = SPLIT_HALF if pairing == "split_half" else INTERLEAVED
        freqs = inverse_frequencies(rot, theta)
        if scaling:
            kind = scaling.get("rope_type", scaling.get("type"))
            if kind == "llama3":
                fac = llama3_factors(freqs, scaling["factor"], scaling["low_freq_factor"],
                                     scaling["high_freq_factor"], scaling["original_max_position_embeddings"])
                freqs = [f / c for f, c in zip(freqs, fac)]
            elif kind == "linear":
                freqs = [f / float(scaling["factor"]) for f in freqs]
            elif kind not in (None, "default"):
                raise ValueError(f"unknown rotary scaling '{kind}'")
        self.freqs = freqs
        self.inv_freq: Optional[torch.Tensor] = None

    def bind(self, get: Callable[[str], Optional[torch.Tensor]], rt: Runtime) -> None:
        super().bind(get, rt)
        self.inv_freq = torch.tensor(self.freqs, dtype=torch.float64, device=rt.device)

    def prepare(self, ctx: StepContext) -> torch.Tensor:
        """(cos, sin) table [T, rot/2, 2] of the step's positions, made once per step."""
        key = ("rotary", id(self))
        table = ctx.shared.get(key)
        if table is None:
            table = K.rope_table(ctx.tok_pos, self.inv_freq)
            ctx.shared[key] = table
        return table
