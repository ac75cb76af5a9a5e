"""What every part of a layer has in common: the tensors it asks for, the runtime it is
bound to, and the description of a step that is handed through the layers.

A part knows its own sizes, constants and tensor names (by a prefix it is given) and
nothing about the model that holds it.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Callable, Dict, List, Optional, Tuple

import torch


@dataclass(frozen=True)
class TensorSpec:
    """One tensor a part reads from the checkpoint.

    kind drives random initialisation: 'matrix' and 'table' N(0, std), 'bias' N(0, std),
    'norm' 1 + U(-0.1, 0.1).  `optional` tensors may be absent."""
    name: str
    shape: Tuple[int, ...]
    kind: str = "matrix"
    optional: bool = False


@dataclass
class Runtime:
    """Where and in which element type a model computes."""
    device: torch.device
    dtype: torch.dtype                  # torch.float32 or torch.bfloat16: matrices, activations, cache
    pack_weights: bool = True           # bfloat16 matrices get a second copy in the matrix cores' order (few-row products)
    pack_budget: Optional[int] = None   # bytes that the packed copies may take together (None: no limit); bind() counts it down

    @property
    def is_f32(self) -> bool:
        return self.dtype == torch.float32


@dataclass(frozen=True)
class KVSpec:
    """Key/value storage a mixer needs for each sequence.  Layers with equal specs share a
    group of the cache; a windowed spec keeps the first `sinks` and the last `window`
    positions of a sequence and gives older pages back."""
    n_kv_heads: int
    head_dim: int
    window: int = 0
    sinks: int = 0


@dataclass(frozen=True)
class StateSpec:
    """Fixed-size state a mixer keeps for each sequence: one tensor of `shape` per slot,
    zeroed when the slot is handed out."""
    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32


@dataclass
class GroupView:
    """A cache group's part of a step: page table rows of the step's sequences."""
    table: torch.Tensor                 # int32 [batch, pages]


@dataclass
class LayerCache:
    """What one scheduled layer sees of the cache in a step."""
    k_pool: Optional[torch.Tensor] = None     # [pages, kv_heads, 64 * head_dim], a page in the matrix cores'
    v_pool: Optional[torch.Tensor] = None     # operand order (cache/pages.py: key_offset, value_offset)
    table: Optional[torch.Tensor] = None      # int32 [batch, pages]
    writes: bool = True                       # False: reads the pages another layer wrote
    state: Optional[torch.Tensor] = None      # [slots, *StateSpec.shape]


@dataclass
class StepContext:
    """One step's batch, on the device and on the host.

    The step's tokens lie one sequence after the other: token t belongs to sequence
    tok_seq[t] (index into the step's batch) and stands at position tok_pos[t]."""
    runtime: Runtime
    n_tokens: int
    batch: int
    ids: torch.Tensor                   # int32 [T]
    tok_seq: torch.Tensor               # int32 [T]
    tok_pos: torch.Tensor               # int32 [T]
    slots: torch.Tensor                 # int32 [B] cache slot of each sequence
    cu_seqlens: List[int]               # host: token offsets of the sequences, B + 1 entries
    starts: List[int]                   # host: position of each sequence's first token in this step
    slot_ids: List[int]                 # host copy of `slots`
    is_decode: bool                     # every sequence brings exactly one token
    max_context: int                    # largest position + 1 in the step (in a graph: the most it may become)
    cu_dev: Optional[torch.Tensor] = None   # int32 [B + 1] token offsets on the device (None in a captured step)
    in_graph: bool = False              # the step is being captured for replay: host lists are not valid
    shared: Dict[object, object] = field(default_factory=dict)   # per-step tables shared by layers
    probe: Optional[Callable[[str], None]] = None                 # called with a part's name when its kernels are queued

    def mark(self, name: str) -> None:
        """A part has queued its kernels (for a step that is timed part by part, engine/probe.py)."""
        if self.probe is not None:
            self.probe(name)


def mark(ctx: Optional[StepContext], name: str) -> None:
    """ctx.mark(name) for a part that may be run without a step around it (ctx None)."""
    if ctx is not None and ctx.probe is not None:
        ctx.probe(name)


class Part:
    """Base of mixers, feed-forwards, norms and position encodings."""

    def tensor_specs(self) -> List[TensorSpec]:
        return []

    def bind(self, get: Callable[[str], Optional[torch.Tensor]], rt: Runtime) -> None:
        """Take the tensors named in tensor_specs() from `get` (host tensors as stored in the
        checkpoint, None for an absent optional one) and keep device copies in the layout
        the kernels want."""
        self.rt = rt

    def weight_bytes(self) -> int:
        """Bytes of the device tensors this part and its sub-parts hold: what a step reads of it."""
        total = 0
        for v in vars(self).values():
            if isinstance(v, torch.Tensor):
                total += v.numel() * v.element_size()
            elif isinstance(v, Part):
                total += v.weight_bytes()
            elif isinstance(v, (list, tuple)):
                total += sum(x.weight_bytes() for x in v if isinstance(x, Part))
        return total

    def packed_bytes(self) -> int:
        """Bytes of the second copies of matrices (in the matrix cores' operand order) that this
        part and its sub-parts hold beside what weight_bytes() counts."""
        total = 0
        for v in vars(self).values():
            if isinstance(v, Part):
                total += v.packed_bytes()
            elif isinstance(v, (list, tuple)):
                total += sum(x.packed_bytes() for x in v if isinstance(x, Part))
        return total

    def matrix_elements(self) -> int:
        """Elements of the matrices this part multiplies every token with (two flops each)."""
        total = 0
        for v in vars(self).values():
            if isinstance(v, Part):
                total += v.matrix_elements()
            elif isinstance(v, (list, tuple)):
                total += sum(x.matrix_elements() for x in v if isinstance(x, Part))
        return total


@dataclass
class Residual:
    """The float32 residual stream x [T, H] offered to a part whose last product may add itself to it,
    with the norm that reads the stream next (None when its rows are not wanted in advance)."""
    x: torch.Tensor
    norm: Optional["Norm"] = None


@dataclass
class NormedRows:
    """A norm's rows that still lack their scale: `squares` holds x * weight in bfloat16 and the sums of
    squares of the rows of x (ops.kernels.RowSquares), left by the product that completed x.  A product
    that takes them applies the scale to its result; tensor() runs the norm's own kernel instead."""
    squares: object
    eps: float
    norm: "Norm"
    x: torch.Tensor

    def tensor(self) -> torch.Tensor:
        return self.norm.forward(self.x)


class Mixer(Part):
    """Token mixer: forward(ctx, h [T, H] in the runtime's type, cache) -> [T, H], or float32
    partial sums [parts, T, H] that the residual sum after it adds.

    Two optional agreements with the block, each announced by a class attribute:
    takes_normed_rows: h may be a NormedRows instead of a tensor;
    adds_to_residual: forward takes `residual=Residual(...)` and may add its output to residual.x
    itself, returning what the product left (ops.kernels.RowSquares) instead of a tensor."""

    takes_normed_rows = False
    adds_to_residual = False

    def kv_spec(self) -> Optional[KVSpec]:
        return None

    def state_spec(self) -> Optional[StateSpec]:
        return None

    # True when forward reads the step only through device tensors (ids, tok_seq, tok_pos, slots,
    # page tables, the state tensor at the rows of `slots`), so that a captured single-token step
    # can be replayed with new contents.  A captured step is run once for real before its
    # capture; the engine puts the fixed-size state back afterwards, so a mixer with state may
    # set this too, as long as the state tensor is all it changes beside its cache pages.
    graph_safe = False

    def forward(self, ctx: StepContext, h: torch.Tensor, cache: LayerCache) -> torch.Tensor:
        raise NotImplementedError


class FeedForward(Part):
    """forward(ctx, h [T, H]) -> [T, H], or float32 partial sums [parts, T, H].  The optional agreements
    of a Mixer (takes_normed_rows, adds_to_residual) hold here too."""

    takes_normed_rows = False
    adds_to_residual = False

    # True when forward launches the same kernels with the same shapes whatever the tokens are
    # (no routing decided on the host), so that a captured single-token step can be replayed.
    graph_safe = False

    def forward(self, ctx: StepContext, h: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError


class Norm(Part):
    """forward(x, delta, rows) -> normed rows in the runtime's type.  `x` is the float32
    residual stream; a pending `delta` ([T, H] or partial sums [parts, T, H]) is added to it
    first (in place).  `delta` may also be what a product that has already added itself to x left
    (ops.kernels.RowSquares): then x is complete, and with `lazy` a norm that can do so returns
    NormedRows for a consumer that takes them."""

    def forward(self, x: torch.Tensor, delta=None, rows: Optional[torch.Tensor] = None,
                write_back: bool = True, lazy: bool = False):
        raise NotImplementedError

    # True when forward takes, as `delta`, what a product that has already added itself to the stream
    # left (ops.kernels.RowSquares).  A block offers the stream to its parts (Residual) only when the
    # norm that reads it next says so.
    takes_row_squares = False

    def row_weight(self) -> Optional[torch.Tensor]:
        """float32 [H]: the weight w of a norm of the form x * w * (a scale of the whole row from the
        row's mean square and eps); None for any other norm."""
        return None


class Block(Part):
    """Arrangement of a layer's parts: which mixers and feed-forwards it holds, with which norms
    around them, and how their outputs join the residual stream.

    forward(ctx, x, pending, caches) -> (x, pending): `x` is the float32 residual stream
    [T, H], `pending` a delta that is still to be added to it ([T, H] or partial sums
    [parts, T, H], or None), `caches` one LayerCache for each of mixers(), in that order.
    `pending` is handed to the block's first norm as its delta and may be whatever that norm takes.

    A block that sets takes_next_norm is also given `next_norm`, the norm that reads the stream after
    this block (entry_norm() of the block that runs next), for parts that prepare its rows."""

    takes_next_norm = False

    def entry_norm(self) -> Optional["Norm"]:
        """The norm that takes `pending` (None if the block has no such norm)."""
        return None

    def mixers(self) -> List["Mixer"]:
        return []

    def feed_forwards(self) -> List["FeedForward"]:
        return []

    def parts(self) -> List[Part]:
        raise NotImplementedError

    def tensor_specs(self) -> List[TensorSpec]:
        return [s for p in self.parts() for s in p.tensor_specs()]

    def bind(self, get: Callable[[str], Optional[torch.Tensor]], rt: Runtime) -> None:
        super().bind(get, rt)
        for p in self.parts():
            p.bind(get, rt)

    def forward(self, ctx: StepContext, x: torch.Tensor, pending: Optional[torch.Tensor],
                caches: List[LayerCache]) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
        raise NotImplementedError


class PositionEncoding(Part):
    """prepare(ctx) -> whatever the mixer's kernels need for this step's positions."""

    def prepare(self, ctx: StepContext):
        raise NotImplementedError

    def weight_bytes(self) -> int:
        return 0                   # its tables come from the configuration, not from the checkpoint


# ---------------------------------------------------------------------------
# registries: a kind name -> the class that builds the part from keyword parameters
# ---------------------------------------------------------------------------
MIXERS: Dict[str, type] = {}
FEED_FORWARDS: Dict[str, type] = {}
NORMS: Dict[str, type] = {}
POSITIONS: Dict[str, type] = {}
BLOCKS: Dict[str, type] = {}


def _register(table: Dict[str, type], what: str):
    def deco(name: str):
        def wrap(cls):
            table[name] = cls
            return cls
        return wrap
    return deco


register_mixer = _register(MIXERS, "mixer")
register_feed_forward = _register(FEED_FORWARDS, "feed-forward")
register_norm = _register(NORMS, "norm")
register_position = _register(POSITIONS, "position encoding")
register_block = _register(BLOCKS, "block")


def make(table: Dict[str, type], what: str, kind: str, **params):
    if kind not in table:
        raise KeyError(f"unknown {what} '{kind}'; known: {sorted(table)}")
    return table[kind](**params)
