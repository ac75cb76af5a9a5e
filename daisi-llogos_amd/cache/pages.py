"""Host-side bookkeeping of the cache: which slots are handed out and which pages each
sequence holds.  No device memory here; the accounting can be tested on its own."""
from __future__ import annotations

from typing import Dict, List

# Positions a page holds.  This is the definition; the kernel library has the same number
# compiled in (kPageTokens) and loading it fails if the two differ.
PAGE_TOKENS = 64
# A page holds a head's keys and values in fragments of 16 dimensions (key_offset, value_offset):
# head sizes are multiples of this, up to the most the attention kernels take.
HEAD_DIM_STEP = 16
MAX_HEAD_DIM = 512


class CacheError(RuntimeError):
    """Misuse of the cache: a slot freed twice, an unknown slot, a page given back twice."""


class CacheFull(CacheError):
    """Not enough free pages (or slots) for what a step asks."""


def key_offset(token: int, d: int, head_dim: int) -> int:
    """Where dimension d of the key at position `token` of a page lies within one kv head's
    part of the page (PAGE_TOKENS * head_dim elements).  Pages are stored in the order in
    which the matrix cores take them as operands: blocks of 4 tokens, then 8 dimensions, then
    16 rows of 8 values, so that a wave's load of a fragment is 1 KB of consecutive memory.
    The kernel library has the same rule compiled in (page_key_offset) and loading it fails
    if the two differ."""
    return ((((token >> 2) & 3) * (head_dim >> 3) + (d >> 3)) * 16 + (((token >> 4) << 2) | (token & 3))) * 8 + (d & 7)


def value_offset(token: int, d: int) -> int:
    """The same for values: 16 dimensions, then halves of 8 tokens, then 16 tokens' groups,
    then 16 rows (dimensions) of 8 consecutive tokens."""
    return ((((d >> 4) * 2 + ((token >> 3) & 1)) * 4 + (token >> 4)) * 16 + (d & 15)) * 8 + (token & 7)


def page_offsets(head_dim: int):
    """(keys, values): two lists [PAGE_TOKENS][head_dim] of element offsets within one kv
    head's part of a page, for code that fills or reads pages on the host (tests, tools)."""
    if head_dim <= 0 or head_dim % 16:
        raise ValueError(f"head size {head_dim} is not a multiple of 16")
    keys = [[key_offset(t, d, head_dim) for d in range(head_dim)] for t in range(PAGE_TOKENS)]
    values = [[value_offset(t, d) for d in range(head_dim)] for t in range(PAGE_TOKENS)]
    return keys, values


def pages_for(n_tokens: int) -> int:
    return (n_tokens + PAGE_TOKENS - 1) // PAGE_TOKENS


class PagePool:
    """Page ids 0..n-1; `take` hands out free ones, `give` takes them back."""

    def __init__(self, n_pages: int):
        if n_pages <= 0:
            raise ValueError("a page pool needs at least one page")
        self.n_pages = n_pages
        self._free: List[int] = list(range(n_pages - 1, -1, -1))     # pop() hands out low ids first
        self._held = [False] * n_pages

    @property
    def free_count(self) -> int:
        return len(self._free)

    def take(self, n: int) -> List[int]:
        if n > len(self._free):
            raise CacheFull(f"{n} pages wanted, {len(self._free)} of {self.n_pages} free")
        out = [self._free.pop() for _ in range(n)]
        for p in out:
            self._held[p] = True
        return out

    def give(self, pages: List[int]) -> None:
        for p in pages:
            if not 0 <= p < self.n_pages or not self._held[p]:
                raise CacheError(f"page {p} is given back but is not held")
            self._held[p] = False
            self._free.append(p)


class SlotAllocator:
    """Slot ids for live sequences; freed slots are handed out again, lowest first."""

    def __init__(self, n_slots: int):
        self.n_slots = n_slots
        self._free: List[int] = list(range(n_slots - 1, -1, -1))
        self._live = [False] * n_slots

    @property
    def free_count(self) -> int:
        return len(self._free)

    @property
    def live(self) -> List[int]:
        return [i for i, l in enumerate(self._live) if l]

    def grow(self, n_slots: int) -> None:
        if n_slots > self.n_slots:
            self._free = list(range(n_slots - 1, self.n_slots - 1, -1)) + self._free
            self._free.sort(reverse=True)
            self._live += [False] * (n_slots - self.n_slots)
            self.n_slots = n_slots

    def alloc(self) -> int:
        if not self._free:
            raise CacheFull(f"all {self.n_slots} slots are in use")
        s = self._free.pop()
        self._live[s] = True
        return s

    def free(self, slot: int) -> None:
        self.check(slot)
        self._live[slot] = False
        self._free.append(slot)
        self._free.sort(reverse=True)

    def check(self, slot: int) -> None:
        if not isinstance(slot, int) or not 0 <= slot < self.n_slots or not self._live[slot]:
            raise CacheError(f"slot {slot} is not in use")


class SequencePages:
    """The pages one sequence holds in one group: page index -> page id, -1 once a page
    has left the window and was given back."""

    def __init__(self):
        self.pages: List[int] = []
        self._row = None                    # the list as an int32 array, made when asked for

    def held(self) -> List[int]:
        return [p for p in self.pages if p >= 0]

    def touched(self) -> None:
        """The list has changed (GroupPages says so after every change it makes)."""
        self._row = None

    def row(self):
        """The list as a numpy int32 array, kept until the list changes: a step's page table is
        put together from these rows, and a sequence's list changes once in PAGE_TOKENS steps."""
        if self._row is None or len(self._row) != len(self.pages):
            import numpy as np
            self._row = np.asarray(self.pages, dtype=np.int32)
        return self._row


class GroupPages:
    """Pages of all live sequences in one cache group (layers with the same storage needs)."""

    def __init__(self, n_pages: int, window: int = 0, sinks: int = 0):
        self.pool = PagePool(n_pages)
        self.window, self.sinks = window, sinks
        self.seqs: Dict[int, SequencePages] = {}

    def open(self, slot: int) -> None:
        if slot in self.seqs:
            raise CacheError(f"slot {slot} is opened twice")
        self.seqs[slot] = SequencePages()

    def close(self, slot: int) -> None:
        if slot not in self.seqs:
            raise CacheError(f"slot {slot} is closed but not open")
        self.pool.give(self.seqs.pop(slot).held())

    def pages_needed(self, slot: int, new_len: int) -> int:
        return max(0, pages_for(new_len) - len(self.seqs[slot].pages))

    def extend(self, slot: int, new_len: int) -> None:
        """Make sure positions below new_len have pages."""
        n = self.pages_needed(slot, new_len)
        if n:
            self.seqs[slot].pages += self.pool.take(n)
            self.seqs[slot].touched()

    def release_behind_window(self, slot: int, length: int) -> int:
        """After the sequence has `length` tokens: a later query at position >= length sees
        keys > position - window, so pages that end at or before length - window are dead,
        except those that hold sink positions.  Returns the number of pages given back."""
        if self.window <= 0:
            return 0
        pages = self.seqs[slot].pages
        dead = []
        for i, p in enumerate(pages):
            last = i * PAGE_TOKENS + PAGE_TOKENS - 1
            if last > length - self.window:
                break
            if p >= 0 and i * PAGE_TOKENS >= self.sinks:
                dead.append(p)
                pages[i] = -1
        self.pool.give(dead)
        if dead:
            self.seqs[slot].touched()
        return len(dead)

    def truncate(self, slot: int, length: int) -> None:
        """Forget positions >= length (pages beyond are given back)."""
        pages = self.seqs[slot].pages
        keep = pages_for(length)
        if self.window > 0 and any(p < 0 for p in pages[:keep]) and length > 0:
            raise CacheError("a windowed group cannot be truncated into pages it has given back")
        self.trim(slot, length)

    def trim(self, slot: int, length: int) -> None:
        """Give back the pages beyond those that `length` positions need (what a step reserved
        and did not come to use)."""
        pages = self.seqs[slot].pages
        keep = pages_for(length)
        self.pool.give([p for p in pages[keep:] if p >= 0])
        del pages[keep:]
        self.seqs[slot].touched()
