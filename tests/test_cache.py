"""The cache's bookkeeping: no slot or page is lost, held twice or freed twice."""
import importlib
import random

import pytest

pages = importlib.import_module("daisi-llogos_amd.cache.pages")
kvc = importlib.import_module("daisi-llogos_amd.cache.kv_cache")
base = importlib.import_module("daisi-llogos_amd.parts.base")


def _cache(max_tokens=64 * 10, windows=(0,), n_slots=2, state=False):
    needs = [(base.KVSpec(2, 16, w, 0), base.StateSpec((4,)) if state else None) for w in windows]
    return kvc.Cache(needs, [None] * len(needs), max_tokens, rt=None, n_slots=n_slots)


def test_page_pool_accounting():
    pool = pages.PagePool(4)
    a = pool.take(3)
    assert sorted(a) == [0, 1, 2] and pool.free_count == 1
    with pytest.raises(pages.CacheFull):
        pool.take(2)
    assert pool.free_count == 1                                         # a refused take takes nothing
    pool.give([a[1]])
    with pytest.raises(pages.CacheError):
        pool.give([a[1]])                                               # given back twice
    with pytest.raises(pages.CacheError):
        pool.give([3])                                                  # never taken
    assert sorted(pool.take(2)) == [1, 3]


def test_slots_are_reused_lowest_first_and_never_freed_twice():
    s = pages.SlotAllocator(3)
    a, b, c = s.alloc(), s.alloc(), s.alloc()
    assert (a, b, c) == (0, 1, 2)
    with pytest.raises(pages.CacheFull):
        s.alloc()
    s.free(b)
    with pytest.raises(pages.CacheError):
        s.free(b)
    with pytest.raises(pages.CacheError):
        s.check(7)
    assert s.alloc() == 1 and s.live == [0, 1, 2]
    s.grow(5)
    assert s.alloc() == 3 and s.alloc() == 4


def test_lengths_pages_and_release():
    c = _cache()
    s0, s1 = c.alloc_slot(), c.alloc_slot()
    c.reserve([s0, s1], [65, 1])
    c.commit([s0, s1], [65, 1])
    assert c.length(s0) == 65 and c.length(s1) == 1 and c.free_pages() == [7]
    t = c.step_tables([s1, s0])[0]
    assert t.shape == (2, 2) and t[0, 1] == -1 and len({t[0, 0], t[1, 0], t[1, 1]}) == 3
    c.reserve([s0], [128]); c.commit([s0], [128])
    assert c.free_pages() == [7]                                        # position 127 is still in page 1
    c.reserve([s0], [129]); c.commit([s0], [129])
    assert c.free_pages() == [6]
    c.free_slot(s0)
    assert c.free_pages() == [9]
    with pytest.raises(pages.CacheError):
        c.free_slot(s0)
    with pytest.raises(pages.CacheError):
        c.length(s0)
    with pytest.raises(pages.CacheError):
        c.reserve([s0], [3])
    assert c.alloc_slot() == s0 and c.length(s0) == 0                   # the slot comes back empty


def test_reserve_is_all_or_nothing():
    c = _cache(max_tokens=64 * 3)
    a, b = c.alloc_slot(), c.alloc_slot()
    with pytest.raises(pages.CacheFull):
        c.reserve([a, b], [64, 129])
    assert c.free_pages() == [3]
    c.reserve([a, b], [64, 128])
    assert c.free_pages() == [0]


def test_slots_grow_on_demand():
    c = _cache(n_slots=1)
    got = [c.alloc_slot() for _ in range(5)]
    assert got == [0, 1, 2, 3, 4]


def test_groups_have_their_own_pages_and_windows_give_back():
    c = _cache(max_tokens=64 * 8, windows=(0, 70, 70))
    assert len(c.groups) == 2 and c.entry_group == [(0, 0), (1, 0), (1, 1)]
    s = c.alloc_slot()
    c.reserve([s], [300]); c.commit([s], [300])
    # full group holds 5 pages; the window group keeps positions > 300 - 70 = 230: pages 3, 4
    assert c.free_pages() == [3, 6]
    assert list(c.step_tables([s])[1][0]) == [-1, -1, -1] + list(c.groups[1].pages.seqs[s].pages[3:])
    c.free_slot(s)
    assert c.free_pages() == [8, 8]


def test_sinks_keep_their_pages():
    g = pages.GroupPages(10, window=64, sinks=4)
    g.open(0)
    g.extend(0, 400)
    g.release_behind_window(0, 400)
    kept = [i for i, p in enumerate(g.seqs[0].pages) if p >= 0]
    assert kept == [0, 5, 6]                                            # page 0 holds the sinks; 337.. live in 5, 6


def test_truncate():
    c = _cache()
    s = c.alloc_slot()
    c.reserve([s], [200]); c.commit([s], [200])
    c.truncate(s, 64)
    assert c.length(s) == 64 and c.free_pages() == [9]
    with pytest.raises(pages.CacheError):
        c.truncate(s, 65)
    st = _cache(state=True)
    s = st.alloc_slot()
    st.reserve([s], [10]); st.commit([s], [10])
    with pytest.raises(pages.CacheError, match="state"):
        st.truncate(s, 5)


def test_random_traffic_never_loses_or_doubles_a_page():
    rnd = random.Random(1)
    c = _cache(max_tokens=64 * 40, windows=(0, 100), n_slots=4)
    live = {}
    for _ in range(2000):
        op = rnd.random()
        if op < 0.25 and len(live) < 12:
            live[c.alloc_slot()] = 0
        elif op < 0.45 and live:
            s = rnd.choice(list(live))
            c.free_slot(s)
            del live[s]
        elif live:
            batch = rnd.sample(list(live), rnd.randint(1, len(live)))
            lens = [live[s] + rnd.choice([1, 1, 1, 30, 90]) for s in batch]
            try:
                c.reserve(batch, lens)
            except pages.CacheFull:
                continue
            c.commit(batch, lens)
            for s, n in zip(batch, lens):
                live[s] = n
        for g in c.groups:
            held = [p for sp in g.pages.seqs.values() for p in sp.held()]
            assert len(held) == len(set(held))                          # no page held twice
            assert len(held) + g.pages.pool.free_count == g.pages.pool.n_pages   # none lost
            assert set(g.pages.seqs) == set(live)
        assert sorted(c.live_slots) == sorted(live)
        for s, n in live.items():
            assert c.length(s) == n
            assert len(c.groups[0].pages.seqs[s].pages) == pages.pages_for(n)


@pytest.mark.parametrize("hd", [16, 48, 64, 128, 256])
def test_a_page_holds_every_element_once_and_a_fragment_is_one_run_of_memory(hd):
    """The page layout is a rule of its own (the kernels have a copy of it): every (token,
    dimension) has a place of its own inside the kv head's part of the page, and the eight
    values a lane of the matrix cores takes lie together, the 64 lanes of a fragment one after
    the other: keys, lane (i, g) of fragment (rb, sk) = dimensions 32 sk + 8 g .. + 7 of token
    16 (i / 4) + 4 rb + i % 4; values, lane (i, g) of fragment (db, half) = tokens
    16 g + 8 half .. + 7 of dimension 16 db + i."""
    keys, values = pages.page_offsets(hd)
    for table in (keys, values):
        flat = sorted(x for row in table for x in row)
        assert flat == list(range(pages.PAGE_TOKENS * hd))
    for rb in range(4):
        for piece in range(hd // 8):                                    # eight dimensions of 16 rows: 256 bytes in bfloat16
            for i in range(16):
                token = 16 * (i // 4) + 4 * rb + i % 4
                want = ((rb * (hd // 8) + piece) * 16 + i) * 8
                assert [keys[token][8 * piece + e] for e in range(8)] == list(range(want, want + 8))
        for sk in range(hd // 32 if hd % 32 == 0 else 0):               # four pieces are a fragment of the matrix cores
            for lane in range(64):
                i, g = lane & 15, lane >> 4
                assert keys[16 * (i // 4) + 4 * rb + i % 4][32 * sk + 8 * g] == ((rb * (hd // 32) + sk) * 64 + lane) * 8
    for db in range(hd // 16):
        for half in range(2):
            for lane in range(64):
                i, g = lane & 15, lane >> 4
                want = ((2 * db + half) * 64 + lane) * 8
                assert [values[16 * g + 8 * half + e][16 * db + i] for e in range(8)] == list(range(want, want + 8))
    with pytest.raises(ValueError):
        pages.page_offsets(40)


def test_unreserve_gives_back_what_a_step_reserved_and_nothing_else():
    c = _cache(max_tokens=64 * 8, windows=(0, 64), n_slots=2)
    a, b = c.alloc_slot(), c.alloc_slot()
    c.reserve([a], [200]); c.commit([a], [200])                             # the windowed group gives pages back at once
    free = c.free_pages()
    held = [list(g.pages.seqs[a].pages) for g in c.groups]
    c.reserve([a, b], [260, 70])
    assert c.free_pages() != free
    c.unreserve([a, b])
    assert c.free_pages() == free and c.length(a) == 200 and c.length(b) == 0
    assert [list(g.pages.seqs[a].pages) for g in c.groups] == held
    assert all(g.pages.seqs[b].pages == [] for g in c.groups)
    t = c.step_tables([a, b])                                               # rows follow the lists after every change
    assert [list(r[0][:len(h)]) for r, h in zip(t, held)] == held
    c.free_slot(a); c.free_slot(b)
    assert c.free_pages() == [g.pages.pool.n_pages for g in c.groups]
