"""The cache of a model: paged key/value storage in groups, fixed-size state per slot,
and the lengths of the live sequences.

The reference keeps one cache object per sequence, two tensors [kv heads, max positions,
head size] per attention layer with one `Length`, and a separate per-layer state object
for mixers with fixed-size state (Daisi.Llogos/Inference/KvCache.cs:8-71, 90-108, 135-136;
Daisi.Llogos/Inference/DeltaNetState.cs).  Here sequences share one store: a sequence
takes a slot, its keys and values live in pages of 64 positions, layers whose mixers ask
for the same storage (kv heads, head size, window) form a group with its own pages, and
a slot's pages go back to the pool when the slot is freed."""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

from ..parts.base import KVSpec, LayerCache, Runtime, StateSpec
from .pages import PAGE_TOKENS, CacheError, CacheFull, GroupPages, SlotAllocator, pages_for


class KVGroup:
    def __init__(self, spec: KVSpec, entries: List[int], n_pages: int, rt: Optional[Runtime]):
        self.spec = spec
        self.entries = entries                       # units that own storage here
        self.pages = GroupPages(n_pages, spec.window, spec.sinks)
        self.k = self.v = None
        if rt is not None:
            # a kv head's part of a page is PAGE_TOKENS * head size elements in the matrix cores'
            # operand order (pages.key_offset, pages.value_offset); one page more than the pool
            # hands out: the page of padding rows (Cache.pad_page)
            shape = (len(entries), n_pages + 1, spec.n_kv_heads, PAGE_TOKENS * spec.head_dim)
            self.k = torch.zeros(shape, dtype=rt.dtype, device=rt.device)
            self.v = torch.zeros(shape, dtype=rt.dtype, device=rt.device)

    def bytes(self) -> int:
        return 0 if self.k is None else 2 * self.k.numel() * self.k.element_size()


class Cache:
    """needs: per unit (one mixer of one scheduled run of a layer) a pair (KVSpec or None,
    StateSpec or None), as Model.cache_needs() gives them; reads_from: per unit the unit whose
    storage it reads (None or itself when it owns), as Model.cache_reads() gives them.
    With rt=None no device memory is made (bookkeeping only)."""

    def __init__(self, needs: Sequence[Tuple[Optional[KVSpec], Optional[StateSpec]]],
                 reads_from: Sequence[Optional[int]], max_tokens: int, rt: Optional[Runtime],
                 n_slots: int = 64):
        self.rt = rt
        self.n_pages = max(1, pages_for(max_tokens))
        self.slots = SlotAllocator(n_slots)
        self.lengths: Dict[int, int] = {}
        self.groups: List[KVGroup] = []
        self.entry_group: List[Optional[Tuple[int, int]]] = [None] * len(needs)   # entry -> (group, index in group)
        by_spec: Dict[KVSpec, List[int]] = {}
        for e, (kv, _) in enumerate(needs):
            if kv is not None:
                by_spec.setdefault(kv, []).append(e)
        for spec, entries in by_spec.items():
            g = len(self.groups)
            self.groups.append(KVGroup(spec, entries, self.n_pages, rt))
            for i, e in enumerate(entries):
                self.entry_group[e] = (g, i)
        for e, src in enumerate(reads_from):
            if src is not None and src != e:
                self.entry_group[e] = self.entry_group[src]
        self.reads_from = list(reads_from)
        self.state_specs: List[Optional[StateSpec]] = [st for _, st in needs]
        self.states: List[Optional[torch.Tensor]] = [None] * len(needs)
        if rt is not None:
            for e, st in enumerate(self.state_specs):
                if st is not None:
                    # one row more than there are slots: the state of padding rows (pad_slot)
                    self.states[e] = torch.zeros((n_slots + 1,) + tuple(st.shape), dtype=st.dtype, device=rt.device)

    # ---- slots ------------------------------------------------------------------
    def alloc_slot(self) -> int:
        if self.slots.free_count == 0:
            self._grow_slots(self.slots.n_slots * 2)
        slot = self.slots.alloc()
        self.lengths[slot] = 0
        for g in self.groups:
            g.pages.open(slot)
        for st in self.states:
            if st is not None:
                st[slot].zero_()
        return slot

    def free_slot(self, slot: int) -> None:
        self.slots.free(slot)                        # raises on an unknown or already freed slot
        del self.lengths[slot]
        for g in self.groups:
            g.pages.close(slot)

    def _grow_slots(self, n_slots: int) -> None:
        old = self.slots.n_slots
        self.slots.grow(n_slots)
        for e, st in enumerate(self.states):
            if st is not None:
                bigger = torch.zeros((n_slots + 1,) + tuple(st.shape[1:]), dtype=st.dtype, device=st.device)
                bigger[:old].copy_(st[:old])
                self.states[e] = bigger

    # A step that is replayed from a captured graph may carry rows that belong to no sequence, so
    # that a few captured batch sizes serve every batch.  Such a row writes its key, value and
    # state somewhere nobody reads: a page and a state row that are never handed out.
    @property
    def pad_slot(self) -> int:
        return self.slots.n_slots

    @property
    def pad_page(self) -> int:
        return self.n_pages

    def length(self, slot: int) -> int:
        self.slots.check(slot)
        return self.lengths[slot]

    @property
    def live_slots(self) -> List[int]:
        return self.slots.live

    def free_pages(self) -> List[int]:
        return [g.pages.pool.free_count for g in self.groups]

    def bytes(self) -> int:
        return sum(g.bytes() for g in self.groups)

    def bytes_per_position(self) -> int:
        """Bytes of keys and values that one position of one sequence takes in all groups."""
        if self.rt is None:
            return 0
        elt = torch.empty((), dtype=self.rt.dtype).element_size()
        return sum(2 * len(g.entries) * g.spec.n_kv_heads * g.spec.head_dim * elt for g in self.groups)

    # ---- a step's storage ----------------------------------------------------------
    def reserve(self, slot_ids: Sequence[int], new_lens: Sequence[int]) -> None:
        """Pages for every position below new_len of each sequence, in every group; either
        all of it or nothing (CacheFull)."""
        for slot in slot_ids:
            self.slots.check(slot)
        for g in self.groups:
            need = sum(g.pages.pages_needed(s, n) for s, n in zip(slot_ids, new_lens))
            if need > g.pages.pool.free_count:
                raise CacheFull(f"the step needs {need} more pages of {PAGE_TOKENS} positions, "
                                f"{g.pages.pool.free_count} of {g.pages.pool.n_pages} are free")
        for g in self.groups:
            for s, n in zip(slot_ids, new_lens):
                g.pages.extend(s, n)

    def unreserve(self, slot_ids: Sequence[int]) -> None:
        """The step did not run: the pages that reserve added beyond each sequence's length go
        back to their pools."""
        for g in self.groups:
            for s in slot_ids:
                g.pages.trim(s, self.lengths[s])

    def commit(self, slot_ids: Sequence[int], new_lens: Sequence[int]) -> None:
        """The step has run: the sequences are new_len long; windowed groups give back the
        pages that no later query can see."""
        for s, n in zip(slot_ids, new_lens):
            self.lengths[s] = n
            for g in self.groups:
                g.pages.release_behind_window(s, n)

    def truncate(self, slot: int, length: int) -> None:
        """Forget a sequence's positions from `length` on (reference: IKvCache.SetLength,
        Daisi.Llogos/Inference/IKvCache.cs:54).  Refused when the model keeps fixed-size
        state, which cannot be rolled back."""
        self.slots.check(slot)
        if not 0 <= length <= self.lengths[slot]:
            raise CacheError(f"cannot truncate slot {slot} of length {self.lengths[slot]} to {length}")
        if any(st is not None for st in self.state_specs) and length != self.lengths[slot]:
            raise CacheError("sequences of a model with fixed-size state cannot be truncated")
        for g in self.groups:
            g.pages.truncate(slot, length)
        self.lengths[slot] = length

    def step_tables(self, slot_ids: Sequence[int]) -> List[np.ndarray]:
        """Per group an int32 array [batch, pages]: page ids of the step's sequences by page
        index, -1 where a sequence has no page."""
        out = []
        for g in self.groups:
            rows = [g.pages.seqs[s].row() for s in slot_ids]
            width = max(1, max(len(r) for r in rows))
            t = np.full((len(rows), width), -1, dtype=np.int32)
            for i, r in enumerate(rows):
                t[i, :len(r)] = r
            out.append(t)
        return out

    def layer_caches(self, tables: List[torch.Tensor]) -> List[LayerCache]:
        """What each unit sees in a step whose group tables are on the device."""
        out = []
        for e, loc in enumerate(self.entry_group):
            lc = LayerCache(state=self.states[e])
            if loc is not None:
                g, i = loc
                grp = self.groups[g]
                lc.k_pool, lc.v_pool, lc.table = grp.k[i], grp.v[i], tables[g]
                lc.writes = self.reads_from[e] is None or self.reads_from[e] == e
            out.append(lc)
        return out
