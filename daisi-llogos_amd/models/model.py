"""A model is data: an embedding table, a list of layers built from parts, the order in
which the layers run, a final norm and an output head."""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Callable, Dict, List, Optional, Tuple

import torch

from ..ops import kernels as K
from ..parts.base import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, KVSpec, LayerCache, Mixer, Part, Runtime, StateSpec,
                          StepContext, TensorSpec, make)
from ..parts.linear import Linear, _to_device


@dataclass
class LayerSpec:
    """Kinds and parameters of one layer's parts.  The four named fields are the parts of the
    pre-norm block; a block of another arrangement (two mixers side by side, a mixer alone)
    names its parts in `more`: keyword of the block's constructor -> (registry, kind,
    parameters) with registry one of 'mixer', 'feed_forward', 'norm', or a list of such triples."""
    mixer: Optional[Tuple[str, dict]] = None
    ffn: Optional[Tuple[str, dict]] = None
    mixer_norm: Optional[Tuple[str, dict]] = None
    ffn_norm: Optional[Tuple[str, dict]] = None
    block: str = "pre_norm"
    more: Dict[str, object] = field(default_factory=dict)


@dataclass(frozen=True)
class ScheduleEntry:
    """One run of a layer.  `cache_of` names an earlier schedule entry whose keys and
    values this run reads instead of writing its own (mixer by mixer, for a block that has
    several); None gives the run a cache of its own."""
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
    embed_scale: float = 1.0       # the embedding rows are multiplied by this (1: a row copy)
    logit_scale: float = 1.0       # the logits are multiplied by this ...
    logit_softcap: float = 0.0     # ... and then, if > 0, bent to cap * tanh(logit / cap)


_REGISTRIES = {"mixer": (MIXERS, "mixer"), "feed_forward": (FEED_FORWARDS, "feed-forward"), "norm": (NORMS, "norm")}


def _make_part(triple):
    registry, kind, params = triple
    if registry not in _REGISTRIES:
        raise KeyError(f"unknown kind of part '{registry}'; known: {sorted(_REGISTRIES)}")
    table, what = _REGISTRIES[registry]
    return make(table, what, kind, **params)


def build_layer(spec: LayerSpec):
    built = {}
    for key, (registry, pair) in (("mixer", ("mixer", spec.mixer)), ("ffn", ("feed_forward", spec.ffn)),
                                  ("mixer_norm", ("norm", spec.mixer_norm)), ("ffn_norm", ("norm", spec.ffn_norm))):
        if pair is not None:
            built[key] = _make_part((registry, pair[0], pair[1]))
    for key, what in spec.more.items():
        built[key] = [_make_part(t) for t in what] if isinstance(what, list) else _make_part(what)
    return make(BLOCKS, "block", spec.block, **built)


class Model:
    """Built from a ModelSpec; bound to device tensors by `bind`; `forward` runs one step.

    The cache is asked for by *unit*: one unit for each mixer of each scheduled run, in the
    order of the schedule and, within a run, of the block's mixers()."""

    def __init__(self, spec: ModelSpec):
        self.spec = spec
        self.layers = [build_layer(ls) for ls in spec.layers]
        self.final_norm = make(NORMS, "norm", spec.final_norm[0], **spec.final_norm[1])
        self.schedule = list(spec.schedule) if spec.schedule is not None else \
            [ScheduleEntry(i) for i in range(len(self.layers))]
        self.entry_units: List[List[int]] = []               # schedule entry -> its units
        self.unit_mixers: List[Mixer] = []
        for e in self.schedule:
            if not 0 <= e.layer < len(self.layers):
                raise ValueError(f"a schedule entry names layer {e.layer}, the model has {len(self.layers)}")
            mixers = self.layers[e.layer].mixers()
            self.entry_units.append(list(range(len(self.unit_mixers), len(self.unit_mixers) + len(mixers))))
            self.unit_mixers += mixers
        self._check_schedule()
        self.head = Linear([spec.head_name], spec.hidden_size, [spec.vocab_size])
        self.embed_table: Optional[torch.Tensor] = None
        self.rt: Optional[Runtime] = None

    def _check_schedule(self) -> None:
        for i, e in enumerate(self.schedule):
            if e.cache_of is not None:
                if not 0 <= e.cache_of < i:
                    raise ValueError(f"schedule entry {i} reads the cache of entry {e.cache_of}, which does not run before it")
                src = self.schedule[e.cache_of]
                if src.cache_of is not None:
                    raise ValueError(f"schedule entry {i} must read from an entry that owns its cache")
                mine = [m.kv_spec() for m in self.layers[e.layer].mixers()]
                theirs = [m.kv_spec() for m in self.layers[src.layer].mixers()]
                if mine != theirs:
                    raise ValueError(f"schedule entry {i} and entry {e.cache_of} need different key/value storage")

    @property
    def graph_safe(self) -> bool:
        """Whether single-token steps can be captured and replayed: every mixer and feed-forward says so."""
        return all(m.graph_safe for layer in self.layers for m in layer.mixers()) and \
            all(getattr(f, "graph_safe", False) for layer in self.layers for f in layer.feed_forwards())

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
        """Per unit: key/value storage (None when it reads another run's or needs none) and
        fixed-size state."""
        needs = []
        for e, units in zip(self.schedule, self.entry_units):
            for u in units:
                mixer = self.unit_mixers[u]
                needs.append((mixer.kv_spec() if e.cache_of is None else None, mixer.state_spec()))
        return needs

    def cache_reads(self) -> List[Optional[int]]:
        """Per unit: the unit whose keys and values it reads, None when it owns its storage."""
        reads: List[Optional[int]] = []
        for e, units in zip(self.schedule, self.entry_units):
            for j, _ in enumerate(units):
                reads.append(None if e.cache_of is None else self.entry_units[e.cache_of][j])
        return reads

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

    def describe(self) -> str:
        """One line about the built model, from its own parts: layers, widths, vocabulary, and the
        heads of the mixers that have any (no field of an architecture's configuration is asked for)."""
        s = self.spec
        text = f"{len(self.layers)} layers"
        if len(self.schedule) != len(self.layers):
            text += f" in {len(self.schedule)} runs"
        text += f", hidden {s.hidden_size}"
        heads = sorted({(m.n_heads, getattr(m, "n_kv_heads", m.n_heads)) for m in self.unit_mixers if hasattr(m, "n_heads")})
        if heads:
            text += ", " + " and ".join(f"{q}/{kv}" for q, kv in heads) + " heads"
        return text + f", vocab {s.vocab_size}"

    # ---- what a step costs -----------------------------------------------------
    def step_weight_bytes(self) -> int:
        """Bytes of weights a step reads once: every scheduled run of a layer, the final norm and
        the head (of the embedding table a step reads a row a token, which is not counted)."""
        runs = sum(self.layers[e.layer].weight_bytes() for e in self.schedule)
        return runs + self.final_norm.weight_bytes() + self.head.weight_bytes()

    def packed_weight_bytes(self) -> int:
        """Bytes of device memory that the packed second copies of the matrices take (each layer once)."""
        return sum(layer.packed_bytes() for layer in self.layers) + self.head.packed_bytes()

    def step_flops(self, lens: List[int], starts: Optional[List[int]] = None, wanted_rows: int = 0) -> float:
        """Floating-point operations of a step that brings lens[i] tokens to sequence i, which
        already holds starts[i]: two per matrix element and token; for mixers that say how wide
        their heads are (n_heads, head_dim), the products with the keys and with the values over
        the causal half of the score matrix; the head on the wanted rows."""
        starts = starts or [0] * len(lens)
        tokens = sum(lens)
        total = 2.0 * tokens * sum(self.layers[e.layer].matrix_elements() for e in self.schedule)
        pairs = sum(n * s + n * (n + 1) / 2.0 for n, s in zip(lens, starts))        # (query, visible key) pairs
        for m in self.unit_mixers:
            if hasattr(m, "n_heads") and hasattr(m, "head_dim"):
                total += 4.0 * m.n_heads * m.head_dim * pairs
        return total + 2.0 * wanted_rows * self.head.matrix_elements()

    # ---- one step ---------------------------------------------------------------
    def forward(self, ctx: StepContext, caches: List[LayerCache], want_rows: Optional[torch.Tensor]) -> Optional[torch.Tensor]:
        """Runs the step's tokens through the scheduled layers; `caches` holds one LayerCache for
        each unit.  Returns float32 logits [len(want_rows), vocab] for the wanted token rows, or
        None when nothing is wanted."""
        s = self.spec
        x = K.embed(self.embed_table, ctx.ids, s.embed_scale)
        ctx.mark("embed")
        pending = None
        blocks = [self.layers[entry.layer] for entry in self.schedule]
        for i, (block, units) in enumerate(zip(blocks, self.entry_units)):
            if block.takes_next_norm:
                # the norm that reads the stream after this block: the next block's first one, the final
                # norm after the last (None: the next block has no such norm and takes `pending` as a tensor)
                next_norm = blocks[i + 1].entry_norm() if i + 1 < len(blocks) else self.final_norm
                x, pending = block.forward(ctx, x, pending, [caches[u] for u in units], next_norm=next_norm)
            else:
                x, pending = block.forward(ctx, x, pending, [caches[u] for u in units])
        if want_rows is None or want_rows.numel() == 0:
            return None
        n = self.final_norm.forward(x, pending, rows=want_rows, write_back=False)
        ctx.mark("norm")
        logits = self.head.forward(n, out_dtype=torch.float32)
        ctx.mark("head")
        if s.logit_scale != 1.0 or s.logit_softcap > 0.0:
            K.scale_softcap(logits, s.logit_scale, s.logit_softcap)
        return logits
