"""The step function: a batch of sequences, each with its next tokens, run as one batch
from the cache; logits come back for the wanted places.

The reference has two step shapes for one sequence: a whole prompt
(ForwardBatchedPrefill, Daisi.Llogos/Inference/ForwardPass.cs:630-697) and one token
(Forward, :174-184).  Here a step takes any number of sequences with unequal token
counts; sequences are not padded to a common length.  (A replayed single-token step may
carry whole rows that belong to no sequence, see graph.py; no kernel mixes rows.)"""
from __future__ import annotations

import os
from typing import List, Optional, Sequence, Tuple, Union

import numpy as np
import torch

from ..cache.kv_cache import Cache
from ..config.model_config import read_config_json
from ..config.registry import architecture_of
from ..models.model import Model
from ..ops import kernels as K
from ..ops import library
from ..parts.base import Runtime, StepContext
from ..weights.loader import Checkpoint
from .graph import GraphCache

_DTYPES = {"float32": torch.float32, "fp32": torch.float32, "f32": torch.float32,
           "bfloat16": torch.bfloat16, "bf16": torch.bfloat16}


GRAPH_MAX_BATCH = 64


class StepError(ValueError):
    """A step that cannot run: empty token list, token out of range, slot used twice, a sequence
    longer than the engine's limit."""


def resolve_dtype(dtype: Union[str, torch.dtype]) -> torch.dtype:
    if isinstance(dtype, torch.dtype):
        if dtype not in (torch.float32, torch.bfloat16):
            raise ValueError(f"dtype {dtype} is not supported (float32 or bfloat16)")
        return dtype
    try:
        return _DTYPES[str(dtype).lower()]
    except KeyError:
        raise ValueError(f"dtype '{dtype}' is not supported (float32 or bfloat16)") from None


def packed_weight_budget(model: Model, dtype: torch.dtype, max_tokens: int, device: torch.device) -> int:
    """Bytes that the packed copies of the bfloat16 matrices may take (the few-row products stream
    a packed copy a quarter faster; prompts need the row-major one): what is free on the GPU now,
    when the model is about to be bound, less the matrices themselves and the cache, which are
    still to be allocated, and less a margin of 15 % of the GPU's memory for activations and
    workspaces.  At the Llama-3.1-70B sizes, 141 GB of matrices, about two thirds of the layers get
    their packed copy; smaller models all.  Whatever else lives on the GPU (another engine in the
    same process, another process) is not counted on: only free memory is."""
    if dtype != torch.bfloat16:
        return 0
    element = torch.empty((), dtype=dtype).element_size()
    elements = 0
    for spec in model.tensor_specs():
        if spec.kind in ("matrix", "table"):
            n = 1
            for d in spec.shape:
                n *= int(d)
            elements += n
    cache = max_tokens * sum(2 * kv.n_kv_heads * kv.head_dim * element for kv, _ in model.cache_needs() if kv is not None)
    with torch.cuda.device(device):
        free, total = torch.cuda.mem_get_info()
        free += torch.cuda.memory_reserved() - torch.cuda.memory_allocated()      # what torch holds but does not use
    return max(0, int(free - 0.15 * total) - element * elements - cache)


def _packing(rt: Runtime, model: Model, max_tokens: int, pack_weights: Optional[bool]) -> None:
    """pack_weights None: packed copies as far as the GPU's memory allows; True: all; False: none."""
    rt.pack_weights = pack_weights is not False and rt.dtype == torch.bfloat16
    rt.pack_budget = packed_weight_budget(model, rt.dtype, max_tokens, rt.device) if pack_weights is None else None


def require_gpu(device: Union[str, torch.device] = "cuda:0") -> torch.device:
    """The device the engine runs on.  There is no CPU path: without a GPU or without the
    kernel library this raises."""
    device = torch.device(device)
    if device.type != "cuda" or not torch.cuda.is_available():
        raise RuntimeError("the engine runs on an AMD GPU only (no CPU fallback); no GPU is visible")
    library.load()
    return device


class Engine:
    """A bound model with its cache.  `step` is the only way tokens reach the model."""

    def __init__(self, model: Model, rt: Runtime, max_tokens: int, n_slots: int = 64, config=None,
                 use_graphs: Optional[bool] = None, max_seq: Optional[int] = None, architecture: str = ""):
        self.model, self.rt, self.config = model, rt, config
        self.architecture = architecture or type(model).__name__      # the registry name the model was built under
        # The longest a sequence may become: the caller's limit (the reference's --max-context,
        # Daisi.Llogos.Cli/Program.cs:194-197, 805) within the positions the model was made for
        # (max_position_embeddings); a step that would go beyond is refused, nothing runs.
        limits = [int(n) for n in (max_seq, model.spec.max_position) if n]
        self.max_seq: Optional[int] = min(limits) if limits else None
        # single-token steps are replayed as HIP graphs when every mixer and feed-forward allows it
        graph_ok = model.graph_safe
        if use_graphs is None:
            use_graphs = os.environ.get("LLOGOS_GRAPHS", "1") != "0"
        self.graphs = GraphCache(self) if (use_graphs and graph_ok) else None
        self.cache = Cache(model.cache_needs(), model.cache_reads(), max_tokens, rt, n_slots)
        self.vocab_size = model.spec.vocab_size
        self.steps_run = 0

    # ---- construction ---------------------------------------------------------------
    @classmethod
    def from_folder(cls, folder: str, dtype: Union[str, torch.dtype] = "bfloat16", max_tokens: int = 4096,
                    n_slots: int = 64, device: Union[str, torch.device] = "cuda:0",
                    use_graphs: Optional[bool] = None, max_seq: Optional[int] = None,
                    pack_weights: Optional[bool] = None, **spec_options) -> "Engine":
        """config.json chooses the model class through the registry; model.safetensors is
        checked against what the model needs before any tensor is read.  pack_weights: None
        gives as many matrices a packed copy as the GPU's memory allows (packed_weight_budget)."""
        dev = require_gpu(device)
        data = read_config_json(folder)
        arch = architecture_of(data)
        config = arch.read_config(data)
        model = Model(arch.model_spec(config, **spec_options))
        ckpt = Checkpoint(folder)
        try:
            tied = model.spec.head_name + ".weight" if model.spec.tie_head else None
            ckpt.check(model.tensor_specs(), tied_head=tied)
            rt = Runtime(dev, resolve_dtype(dtype))
            _packing(rt, model, max_tokens, pack_weights)
            with torch.cuda.device(dev):
                model.bind(ckpt.get, rt)
                torch.cuda.synchronize()
        finally:
            ckpt.close()
        return cls(model, rt, max_tokens, n_slots, config, use_graphs, max_seq, arch.name)

    @classmethod
    def from_config(cls, config: dict, seed: int = 0, dtype: Union[str, torch.dtype] = "bfloat16",
                    max_tokens: int = 4096, n_slots: int = 64, device: Union[str, torch.device] = "cuda:0",
                    std: float = 0.02, use_graphs: Optional[bool] = None, max_seq: Optional[int] = None,
                    pack_weights: Optional[bool] = None, **spec_options) -> "Engine":
        """A model of the parsed config.json `config` with random weights made on the device,
        without a model folder: the weights that write_random_model(folder, config, seed) writes
        (matrices N(0, std), norm weights 1 + U(-0.1, 0.1)), stored in the configuration's
        `torch_dtype` first, as a folder would hold them."""
        from ..weights.random_init import random_tensor, storage_dtype
        dev = require_gpu(device)
        arch = architecture_of(config)
        typed = arch.read_config(config)
        model = Model(arch.model_spec(typed, **spec_options))
        specs = {s.name: s for s in model.tensor_specs()}
        rt = Runtime(dev, resolve_dtype(dtype))
        _packing(rt, model, max_tokens, pack_weights)
        store = storage_dtype(config)

        def get(name: str):
            spec = specs.get(name)
            return None if spec is None else random_tensor(spec, seed, store, std, device=dev)
        with torch.cuda.device(dev):
            model.bind(get, rt)
            torch.cuda.synchronize()
        return cls(model, rt, max_tokens, n_slots, typed, use_graphs, max_seq, arch.name)

    # ---- slots ---------------------------------------------------------------------
    def _graph_slots(self) -> int:
        """Captured graphs hold pointers to the per-slot state tensors, which are made anew
        when the number of slots grows: drop the graphs then."""
        n = self.cache.slots.n_slots
        if getattr(self, "_graphs_for_slots", n) != n and self.graphs is not None:
            self.graphs.clear()
        self._graphs_for_slots = n
        return n

    def alloc_slot(self) -> int:
        return self.cache.alloc_slot()

    def free_slot(self, slot: int) -> None:
        self.cache.free_slot(slot)

    # ---- the step --------------------------------------------------------------------
    # single-token steps can take their token ids from device memory (`device_ids`)
    takes_device_ids = True
    # step(..., borrow=True) may return a buffer that the next step overwrites
    lends_logits = True

    def step(self, entries: Sequence[Tuple[int, Sequence[int]]],
             want: Union[str, Sequence[Sequence[int]], None] = "last",
             device_ids: Optional[Tuple[torch.Tensor, Sequence[int]]] = None,
             borrow: bool = False, probe=None) -> Optional[torch.Tensor]:
        """entries: (slot, next tokens) for each sequence of the batch.  want: 'last', 'all',
        None, or for each entry the places among its tokens whose logits are asked for.
        Returns float32 logits [wanted places, vocab] in the order of the entries and of
        `want`, or None when nothing is wanted.

        device_ids = (ids, rows): every entry brings one token, and entry i's token is
        ids[rows[i]] of an int32 vector on the device (what a sampler wrote after an earlier
        step); the tokens in `entries` are then placeholders.  The host need not know the
        tokens, so the step can be queued while the earlier one still runs.

        borrow: the caller is done with the logits (on the device, in stream order) before it
        asks for the next step, so a replayed step may hand out its own output buffer, which the
        next replay overwrites, instead of a copy (33 MB a step at batch 64 and 128,256 tokens).

        probe: a callable that the model's parts call with their name when their kernels are
        queued (engine/probe.py: StepProbe times the step part by part); such a step is launched
        kernel by kernel, not replayed."""
        if not entries:
            raise StepError("a step needs at least one sequence")
        slot_ids = [int(s) for s, _ in entries]
        if len(set(slot_ids)) != len(slot_ids):
            raise StepError("a slot appears twice in one step")
        counts = [len(t) for _, t in entries]
        if min(counts) <= 0:
            raise StepError("every sequence of a step must bring at least one token")
        ids = np.concatenate([np.asarray(t, dtype=np.int64).reshape(-1) for _, t in entries])
        if ids.min() < 0 or ids.max() >= self.vocab_size:
            raise StepError(f"token id outside 0..{self.vocab_size - 1}")
        if device_ids is not None:
            src, id_rows = device_ids
            if max(counts) != 1 or len(id_rows) != len(entries):
                raise StepError("device_ids needs one token and one row for each sequence")
            if not (isinstance(src, torch.Tensor) and src.dtype == torch.int32 and src.dim() == 1
                    and src.device == self.rt.device):
                raise StepError("device_ids must be an int32 vector on the engine's device")
            if min(id_rows) < 0 or max(id_rows) >= src.numel():
                raise StepError(f"device_ids rows outside 0..{src.numel() - 1}")
        starts = [self.cache.length(s) for s in slot_ids]
        new_lens = [s + c for s, c in zip(starts, counts)]
        if self.max_seq is not None and max(new_lens) > self.max_seq:
            i = int(np.argmax(new_lens))
            raise StepError(f"sequence {i} (slot {slot_ids[i]}) would become {new_lens[i]} positions long; "
                            f"the limit is {self.max_seq}")
        cu = np.zeros(len(entries) + 1, dtype=np.int64)
        np.cumsum(counts, out=cu[1:])
        rows = self._want_rows(want, counts, cu)

        self.cache.reserve(slot_ids, new_lens)
        try:
            logits = self._run(ids, counts, cu, rows, slot_ids, starts, new_lens, device_ids, borrow, probe)
        except BaseException:
            self.cache.unreserve(slot_ids)             # the sequences are as long as before, and hold no page more
            raise
        self.cache.commit(slot_ids, new_lens)
        self.steps_run += 1
        return logits

    def _run(self, ids, counts, cu, rows, slot_ids, starts, new_lens, device_ids, borrow=False, probe=None) -> torch.Tensor:
        T, B = int(cu[-1]), len(counts)
        # (more rows than the hand-written products take would put a library call into the graph)
        if self.graphs is not None and probe is None and T == B and B <= GRAPH_MAX_BATCH and rows == list(range(B)) \
                and self.cache.slots.n_slots == self._graph_slots():
            with torch.cuda.device(self.rt.device):
                logits = self.graphs.step(ids.astype(np.int32), np.asarray(starts, dtype=np.int32),
                                          np.asarray(slot_ids, dtype=np.int32), self.cache.step_tables(slot_ids),
                                          device_ids)
                if not borrow:
                    logits = logits.clone()      # the graph's own buffer is overwritten by its next replay
            return logits
        tok_seq = np.repeat(np.arange(B, dtype=np.int32), counts)
        tok_pos = np.concatenate([np.arange(s, s + c, dtype=np.int32) for s, c in zip(starts, counts)])
        tables = self.cache.step_tables(slot_ids)
        parts = [ids.astype(np.int32), tok_seq, tok_pos, np.asarray(slot_ids, dtype=np.int32),
                 np.asarray(rows, dtype=np.int32), cu.astype(np.int32)] + [t.reshape(-1) for t in tables]
        if device_ids is not None:
            parts.append(np.asarray(device_ids[1], dtype=np.int32))
        dev = self._upload(parts)
        with torch.cuda.device(self.rt.device):
            if device_ids is not None:
                K.gather_i32(dev[0], device_ids[0], dev[-1])
            ctx = StepContext(runtime=self.rt, n_tokens=T, batch=B, ids=dev[0], tok_seq=dev[1], tok_pos=dev[2],
                              slots=dev[3], cu_seqlens=[int(c) for c in cu], starts=starts, slot_ids=slot_ids,
                              is_decode=max(counts) == 1, max_context=max(new_lens), cu_dev=dev[5], probe=probe)
            dev_tables = [d.view(t.shape) for d, t in zip(dev[6:6 + len(tables)], tables)]
            caches = self.cache.layer_caches(dev_tables)
            if probe is not None and hasattr(probe, "context"):
                probe.context(ctx, caches)               # (a probe that wants to run parts of this step again by itself)
            logits = self.model.forward(ctx, caches, dev[4] if len(rows) else None)
        return logits

    def _want_rows(self, want, counts: List[int], cu: np.ndarray) -> List[int]:
        if want is None:
            return []
        if isinstance(want, str):
            if want == "last":
                return [int(cu[i + 1]) - 1 for i in range(len(counts))]
            if want == "all":
                return list(range(int(cu[-1])))
            if want == "none":
                return []
            raise StepError(f"want must be 'last', 'all', 'none' or lists of places, got '{want}'")
        if len(want) != len(counts):
            raise StepError("want must have one list of places for each sequence")
        rows = []
        for i, places in enumerate(want):
            for p in places:
                p = int(p)
                if not 0 <= p < counts[i]:
                    raise StepError(f"wanted place {p} is outside the {counts[i]} tokens of sequence {i}")
                rows.append(int(cu[i]) + p)
        return rows

    def _upload(self, parts: List[np.ndarray]) -> List[torch.Tensor]:
        """One host-to-device copy for all of a step's integer arrays."""
        sizes = [p.size for p in parts]
        flat = np.concatenate(parts) if len(parts) > 1 else parts[0]
        host = torch.from_numpy(np.ascontiguousarray(flat, dtype=np.int32))
        dev = host.to(self.rt.device, non_blocking=False)
        out, o = [], 0
        for n in sizes:
            out.append(dev[o:o + n])
            o += n
        return out
