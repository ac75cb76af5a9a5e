"""A model is data: an embedding table, a list of layers built from parts, the order in
which the layers run, a final norm and an output head."""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Callable, Dict, List, Optional, Tuple

import torch

from ..ops import kernels as K
from ..parts.base import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, KVSpec, LayerCache, Part, Runtime, StateSpec,
                          StepContext, TensorSpec, make)
from ..parts.linear import Linear, _to_device


@dataclass
class LayerSpec:
    """Kinds and parameters of one layer's parts."""
    mixer: Tuple[str, dict]
    ffn: Tuple[str, dict]
    mixer_norm: Tuple[str, dict]
    ffn_norm: Tuple[str, dict]
    block: str = "pre_norm"


@dataclass(frozen=True)
class ScheduleEntry:
    """One run of a layer.  `cache_of` names an earlier schedule entry whose keys and
    values this run reads instead of writing its own; None gives the run a cache of its own."""
    layer: int
    cache_of: Optional[int] = None


@dataclass
class ModelSpec:
    vocab_size: int
    hidden_size: int
    embed_name: str
    layers: List[LayerSpec]
    final_norm: Tuple[str, dict]
    head_name: str
    tie_head: bool = False
    schedule: Optional[List[ScheduleEntry]] = None      # default: every layer once, in order
    eos_token_ids: Tuple[int, ...] = ()
    max_position: int = 0


def build_layer(spec: LayerSpec):
    mixer = make(MIXERS, "mixer", spec.mixer[0], **spec.mixer[1])
    ffn = make(FEED_FORWARDS, "feed-forward", spec.ffn[0], **spec.ffn[1])
    n1 = make(NORMS, "norm", spec.mixer_norm[0], **spec.mixer_norm[1])
    n2 = make(NORMS, "norm", spec.ffn_norm[0], **spec.ffn_norm[1])
    return make(BLOCKS, "block", spec.block, mixer_norm=n1, mixer=mixer, ffn_norm=n2, ffn=ffn)


class Model:
    """Built from a ModelSpec; bound to device tensors by `bind`; `forward` runs one step."""

    def __init__(self, spec: ModelSpec):
        self.spec = spec
        self.layers = [build_layer(ls) for ls in spec.layers]
        self.final_norm = make(NORMS, "norm", spec.final_norm[0], **spec.final_norm[1])
        self.schedule = list(spec.schedule) if spec.schedule is not None else \
            [ScheduleEntry(i) for i in range(len(self.layers))]
        self._check_schedule()
        self.head = Linear([spec.head_name], spec.hidden_size, [spec.vocab_size])
        self.embed_table: Optional[torch.Tensor] = None
        self.rt: Optional[Runtime] = None

    def _check_schedule(self) -> None:
        for i, e in enumerate(self.schedule):
            if not 0 <= e.layer < len(self.layers):
                raise ValueError(f"schedule entry {i} names layer {e.layer}, the model has {len(self.layers)}")
            if e.cache_of is not None:
                if not 0 <= e.cache_of < i:
                    raise ValueError(f"schedule entry {i} reads the cache of entry {e.cache_of}, which does not run before it")
                src = self.schedule[e.cache_of]
                if src.cache_of is not None:
                    raise ValueError(f"schedule entry {i} must read from an entry that owns its cache")
                if self.layers[src.layer].mixer.kv_spec() != self.layers[e.layer].mixer.kv_spec():
                    raise ValueError(f"schedule entry {i} and entry {e.cache_of} need different key/value storage")

    # ---- what the checkpoint must hold ---------------------------------------
    def tensor_specs(self) -> List[TensorSpec]:
        s = self.spec
        specs = [TensorSpec(s.embed_name, (s.vocab_size, s.hidden_size), "table")]
        for layer in self.layers:
            specs += layer.tensor_specs()
        specs += self.final_norm.tensor_specs()
        if not s.tie_head:
            specs.append(TensorSpec(s.head_name + ".weight", (s.vocab_size, s.hidden_size), "matrix"))
        return specs

    # ---- what the cache must hold ---------------------------------------------
    def cache_needs(self) -> List[Tuple[Optional[KVSpec], Optional[StateSpec]]]:
        """Per schedule entry: key/value storage (None when it reads another entry's or needs
        none) and fixed-size state."""
        needs = []
        for e in self.schedule:
            mixer = self.layers[e.layer].mixer
            kv = mixer.kv_spec() if e.cache_of is None else None
            needs.append((kv, mixer.state_spec()))
        return needs

    # ---- binding ---------------------------------------------------------------
    def bind(self, get: Callable[[str], Optional[torch.Tensor]], rt: Runtime) -> None:
        self.rt = rt
        self.embed_table = _to_device([get(self.spec.embed_name)], rt.dtype, rt.device)
        for layer in self.layers:
            layer.bind(get, rt)
        self.final_norm.bind(get, rt)
        if self.spec.tie_head:
            self.head.bind_shared(self.embed_table, rt)      # one allocation serves both
        else:
            self.head.bind(get, rt)

    # ---- one step ---------------------------------------------------------------
    def forward(self, ctx: StepContext, caches: List[LayerCache], want_rows: Optional[torch.Tensor]) -> Optional[torch.Tensor]:
        """Runs the step's tokens through the scheduled layers.  Returns float32 logits
        [len(want_rows), vocab] for the wanted token rows, or None when nothing is wanted."""
        x = K.embed(self.embed_table, ctx.ids)
        pending = None
        for entry, cache in zip(self.schedule, caches):
            x, pending = self.layers[entry.layer].forward(ctx, x, pending, cache)
        if want_rows is None or want_rows.numel() == 0:
            return None
        n = self.final_norm.forward(x, pending, rows=want_rows, write_back=False)
        return self.head.forward(n, out_dtype=torch.float32)
