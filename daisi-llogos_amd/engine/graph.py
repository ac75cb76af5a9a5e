"""Decode steps as HIP graphs.  A step in which every sequence brings one token launches
the same kernels with the same shapes as the last one; only token ids, positions and page
tables change, and those live in device memory.  The step is captured once per batch shape
and replayed, which removes the launch cost of some three hundred kernels per step.

The reference records its single-token forward pass as a CUDA graph and patches it every
token (Daisi.Llogos.Cuda/CudaBackend.cs:99-141); here nothing is patched: the graph reads
what changes from a static buffer that is filled before each replay."""
from __future__ import annotations

import gc
import weakref
from collections import OrderedDict
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

from ..ops import kernels as K
from ..parts.base import StepContext

TABLE_BUCKET = 16          # page-table widths are rounded up to this many pages (1024 positions)
MAX_GRAPHS = 64
# Batch sizes that are captured.  A batch between two of them runs as the next larger one with
# padding rows (token 0 at position 0 of a page and a state row that belong to no sequence),
# so that a batch whose sequences end one after the other does not capture a graph for every
# size on its way down (a capture costs about three replays).  Up to 8 every size is its own;
# above, a size and its bucket are in the same class of row counts of the few-row products
# (16, 32, 64), so a sequence's logits are the same bits with and without the padding.
BATCH_BUCKETS = (1, 2, 3, 4, 5, 6, 7, 8, 12, 16, 24, 32, 48, 64)


def bucket_width(width: int) -> int:
    return -(-max(1, width) // TABLE_BUCKET) * TABLE_BUCKET


def bucket_batch(batch: int) -> int:
    """The captured batch size that serves `batch`.  (The kernel library rounds a batch up the
    same way where a kernel's shape depends on the batch: llogos_batch_class.)"""
    for b in BATCH_BUCKETS:
        if batch <= b:
            return b
    return batch


class DecodeGraph:
    def __init__(self, engine, batch: int, widths: Tuple[int, ...]):
        # no strong reference back to the engine: a graph must die with its engine at once and
        # not later in a collection of reference cycles, which could fall into another capture
        self._engine = weakref.ref(engine)
        self.batch, self.widths = batch, widths
        rt = engine.rt
        B = batch
        # ids, seq, pos, slots, rows, tables, rows of another step's ids to take the ids from
        self.sizes = [B, B, B, B, B] + [B * w for w in widths] + [B]
        total = sum(self.sizes)
        self.host = torch.empty(total, dtype=torch.int32, pin_memory=True)
        self.host_np = self.host.numpy()
        self.dev = torch.zeros(total, dtype=torch.int32, device=rt.device)
        self.views, o = [], 0
        for n in self.sizes:
            self.views.append(self.dev[o:o + n])
            o += n
        self.graph: Optional[torch.cuda.CUDAGraph] = None
        self.logits: Optional[torch.Tensor] = None
        self.copied = torch.cuda.Event()

    def _fill(self, ids, tok_pos, slot_ids, tables: List[np.ndarray], id_rows=None) -> None:
        B = self.batch
        h = self.host_np
        self.copied.synchronize()                  # the last step's copy has left the staging buffer
        h[0:B] = ids
        h[B:2 * B] = np.arange(B, dtype=np.int32)
        h[2 * B:3 * B] = tok_pos
        h[3 * B:4 * B] = slot_ids
        h[4 * B:5 * B] = np.arange(B, dtype=np.int32)
        o = 5 * B
        for t, w in zip(tables, self.widths):
            block = h[o:o + B * w].reshape(B, w)
            block[:, :t.shape[1]] = t
            block[:, t.shape[1]:] = -1
            o += B * w
        h[o:o + B] = id_rows if id_rows is not None else 0
        self.dev.copy_(self.host, non_blocking=True)
        self.copied.record()

    def _forward(self, max_context: int) -> Optional[torch.Tensor]:
        eng, v, B = self._engine(), self.views, self.batch
        ctx = StepContext(runtime=eng.rt, n_tokens=B, batch=B, ids=v[0], tok_seq=v[1], tok_pos=v[2], slots=v[3],
                          cu_seqlens=list(range(B + 1)), starts=[], slot_ids=[], is_decode=True,
                          max_context=max_context, in_graph=True)
        tables = [t.view(B, w) for t, w in zip(v[5:5 + len(self.widths)], self.widths)]
        return eng.model.forward(ctx, eng.cache.layer_caches(tables), v[4])

    def run(self, ids, tok_pos, slot_ids, tables: List[np.ndarray], device_ids=None) -> torch.Tensor:
        """device_ids: (int32 device vector, rows): the step's ids are that vector's values at
        `rows`, picked on the device before the replay, instead of `ids`."""
        if device_ids is None:
            self._fill(ids, tok_pos, slot_ids, tables)
        else:
            self._fill(ids, tok_pos, slot_ids, tables, np.asarray(device_ids[1], dtype=np.int32))
            K.gather_i32(self.views[0], device_ids[0], self.views[-1])
        if self.graph is None:
            # the longest context this graph may ever see: what its page tables can hold
            cap = max(self.widths) * K.PAGE_TOKENS if self.widths else K.PAGE_TOKENS
            # Warm up: lazy workspaces are made outside the capture.  The warm-up is a real run of
            # the step that the replay below runs again.  For keys and values that changes nothing
            # (the same values go to the same places); fixed-size state would be advanced twice,
            # so it is put back.
            states = self._engine().cache.states
            saved = [None if st is None else st.clone() for st in states]
            self._forward(cap)
            for st, keep in zip(states, saved):
                if st is not None:
                    st.copy_(keep)
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            # freeing device memory or another graph is not allowed while a stream captures:
            # keep the collector of reference cycles out of the capture
            gc_was_on = gc.isenabled()
            gc.disable()
            try:
                with torch.cuda.graph(graph):
                    self.logits = self._forward(cap)
            finally:
                if gc_was_on:
                    gc.enable()
            self.graph = graph
        self.graph.replay()
        return self.logits


class GraphCache:
    """Captured decode steps by (batch size, page-table widths); the least recently used
    graph is dropped when there are too many."""

    def __init__(self, engine):
        self._engine = weakref.ref(engine)
        self.graphs: "OrderedDict[tuple, DecodeGraph]" = OrderedDict()

    def clear(self) -> None:
        self.graphs.clear()

    def step(self, ids, tok_pos, slot_ids, tables: List[np.ndarray], device_ids=None) -> torch.Tensor:
        B = len(slot_ids)
        pad = bucket_batch(B) - B
        if pad:
            cache = self._engine().cache
            zeros = np.zeros(pad, dtype=np.int32)
            ids, tok_pos = np.concatenate([ids, zeros]), np.concatenate([tok_pos, zeros])
            slot_ids = np.concatenate([slot_ids, np.full(pad, cache.pad_slot, dtype=np.int32)])
            rows = np.full((pad, 1), cache.pad_page, dtype=np.int32)
            tables = [np.concatenate([t, np.pad(rows, ((0, 0), (0, t.shape[1] - 1)), constant_values=-1)]) for t in tables]
            if device_ids is not None:
                device_ids = (device_ids[0], list(device_ids[1]) + [0] * pad)
        key = (B + pad, tuple(bucket_width(t.shape[1]) for t in tables))
        g = self.graphs.get(key)
        if g is None:
            while len(self.graphs) >= MAX_GRAPHS:
                self.graphs.popitem(last=False)
            g = DecodeGraph(self._engine(), key[0], key[1])
            self.graphs[key] = g
        else:
            self.graphs.move_to_end(key)
        logits = g.run(ids, tok_pos, slot_ids, tables, device_ids)
        return logits[:B] if pad else logits
