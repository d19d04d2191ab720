"""The cache's bookkeeping: no slot or page lost, held twice or freed twice (no GPU)."""
import random

import pytest
import torch

from bitnet_c_amd.cache import PAGE, CacheError, CacheFull, PagedCache, PagePool
from bitnet_c_amd.parts import CacheNeed, KVNeed, StateNeed


def _cache(max_tokens=64 * 8, needs=None, kv_from=None, **kw):
    needs = needs or [CacheNeed(kv=KVNeed(2, 16))] * 2
    return PagedCache(needs, kv_from or [None] * len(needs), max_tokens, dtype=torch.float32, **kw)


def test_page_pool():
    p = PagePool(4)
    a = p.take(3)
    assert sorted(a) == [0, 1, 2] and p.n_free == 1
    with pytest.raises(CacheFull):
        p.take(2)
    p.give_back(a[:1])
    with pytest.raises(CacheError):
        p.give_back(a[:1])                      # freed twice
    with pytest.raises(CacheError):
        p.give_back([7])
    p.check()


def test_slots_and_pages_are_given_back_and_used_again():
    c = _cache()
    a, b = c.alloc_slot(), c.alloc_slot()
    c.reserve([a, b], [65, 1])
    c.commit([a, b], [65, 1])
    assert (c.length(a), c.length(b)) == (65, 1)
    assert c.groups[0].pool.n_free == 8 - 3
    pages_a = list(c.groups[0].pages[a])
    c.reserve([a], [63])                         # 128 positions: still two pages
    c.commit([a], [63])
    assert c.groups[0].pages[a] == pages_a
    c.reserve([a], [1])
    assert len(c.groups[0].pages[a]) == 3
    c.free_slot(a)
    with pytest.raises(CacheError):
        c.free_slot(a)                           # freed twice
    with pytest.raises(CacheError):
        c.length(a)
    assert c.groups[0].pool.n_free == 7
    a2 = c.alloc_slot()
    assert a2 == a and c.length(a2) == 0         # the slot is used again, empty
    c.check()


def test_reserve_is_all_or_nothing():
    c = _cache(max_tokens=64 * 4)
    a, b = c.alloc_slot(), c.alloc_slot()
    c.reserve([a], [64 * 3])
    c.commit([a], [64 * 3])
    before = (list(c.groups[0].pages[a]), list(c.groups[0].pages[b]), c.groups[0].pool.n_free)
    with pytest.raises(CacheFull):
        c.reserve([a, b], [1, 65])               # needs 1 + 2 pages, one is free
    assert (list(c.groups[0].pages[a]), list(c.groups[0].pages[b]), c.groups[0].pool.n_free) == before
    with pytest.raises(CacheError):
        c.reserve([a, a], [1, 1])
    with pytest.raises(CacheError):
        c.reserve([99], [1])
    c.check()


def test_random_traffic_keeps_the_books():
    rnd = random.Random(0)
    c = _cache(max_tokens=64 * 16, max_slots=6)
    live = {}
    for _ in range(2000):
        r = rnd.random()
        if r < 0.3 and c.n_free_slots:
            live[c.alloc_slot()] = 0
        elif r < 0.5 and live:
            s = rnd.choice(list(live))
            c.free_slot(s)
            del live[s]
        elif live:
            ss = rnd.sample(list(live), rnd.randint(1, len(live)))
            ns = [rnd.randint(1, 100) for _ in ss]
            try:
                c.reserve(ss, ns)
                c.commit(ss, ns)
                for s, n in zip(ss, ns):
                    live[s] += n
            except CacheFull:
                pass
        c.check()
        assert {s: c.length(s) for s in c.live_slots()} == live
        held = sum(len(pl) for pl in c.groups[0].pages.values())
        assert held + c.groups[0].pool.n_free == 16


def test_groups_by_need_and_shared_entries():
    full, win = KVNeed(2, 16), KVNeed(2, 16, window=70)
    needs = [CacheNeed(kv=full), CacheNeed(kv=win), CacheNeed(kv=full), CacheNeed(kv=full), CacheNeed()]
    c = _cache(needs=needs, kv_from=[None, None, None, 0, None], max_tokens=64 * 8, device="cpu")
    assert len(c.groups) == 2
    assert c.groups[0].entries == [0, 2] and c.groups[1].entries == [1]     # storage of their own
    assert c.groups[0].k.shape == (2, 8, 2, PAGE, 16) and c.groups[1].k.shape == (1, 8, 2, PAGE, 16)
    assert c.groups[0].v.shape == (2, 8, 2, PAGE, 16)
    cb = PagedCache(needs, [None, None, None, 0, None], 64 * 8, dtype=torch.bfloat16, device="cpu")
    assert cb.groups[0].v.shape == (2, 8, 2, 16, PAGE)          # bfloat16: V transposed inside a page
    tables = {0: torch.zeros(1, 1, dtype=torch.int32), 1: torch.zeros(1, 1, dtype=torch.int32)}
    v0, v3, v4 = c.view(0, tables, 64), c.view(3, tables, 64), c.view(4, tables, 64)
    assert v3.k_pages.data_ptr() == v0.k_pages.data_ptr() and v0.writes and not v3.writes
    assert v4.k_pages is None
    assert c.view(2, tables, 64).k_pages.data_ptr() != v0.k_pages.data_ptr()
    with pytest.raises(CacheError):
        _cache(needs=[CacheNeed(), CacheNeed(kv=full)], kv_from=[None, 0])


def test_a_need_names_the_width_and_the_layout_of_its_values():
    """The layout of a page is the mixer's to say (KVNeed): values of another width than the keys, lying like the
    keys or turned, at either type; needs that differ in it get storage of their own, and an entry cannot read the
    cache of an entry whose layout differs."""
    plain, wide = KVNeed(2, 16), KVNeed(2, 16, v_head_dim=40, v_layout="rows")
    turned, rows = KVNeed(2, 16, v_layout="transposed"), KVNeed(2, 16, v_layout="rows")
    needs = [CacheNeed(kv=n) for n in (plain, wide, turned, rows, wide)]
    for dtype in (torch.float32, torch.bfloat16):
        c = PagedCache(needs, [None] * 5, 64 * 4, dtype=dtype, device="cpu")
        shapes = [(tuple(g.k.shape[2:]), tuple(g.v.shape[2:]), g.v_transposed, g.entries) for g in c.groups]
        own = (2, 16, PAGE) if dtype == torch.bfloat16 else (2, PAGE, 16)      # no layout named: the kernels' for the type
        assert ((2, PAGE, 16), own, dtype == torch.bfloat16, [0]) in shapes
        assert ((2, PAGE, 16), (2, PAGE, 40), False, [1, 4]) in shapes
        # a named layout that is the kernels' own for the type shares no storage with the unnamed need: the need differs
        assert ((2, PAGE, 16), (2, 16, PAGE), True, [2]) in shapes and ((2, PAGE, 16), (2, PAGE, 16), False, [3]) in shapes
        tables = {g: torch.zeros(1, 1, dtype=torch.int32) for g in range(len(c.groups))}
        assert c.view(1, tables, 64).v_transposed is False and c.view(2, tables, 64).v_transposed is True
        assert c.view(1, tables, 64).v_pages.shape == (4, 2, PAGE, 40)
    with pytest.raises(CacheError, match="layouts differ"):
        PagedCache([CacheNeed(kv=wide), CacheNeed(kv=plain)], [None, 0], 64 * 4, device=None)
    with pytest.raises(CacheError, match="layouts differ"):
        PagedCache([CacheNeed(kv=turned), CacheNeed(kv=rows)], [None, 0], 64 * 4, device=None)
    with pytest.raises(ValueError):
        KVNeed(2, 16, v_layout="columns")


def test_window_group_gives_pages_back_while_the_sequence_grows():
    full, win = KVNeed(1, 8), KVNeed(1, 8, window=70)
    c = _cache(needs=[CacheNeed(kv=full), CacheNeed(kv=win)], max_tokens=64 * 10)
    s = c.alloc_slot()
    for _ in range(8):
        c.reserve([s], [64])
        c.commit([s], [64])
        c.check()
    assert c.groups[0].pool.n_free == 2                    # all keys: 8 pages held
    held = [p for p in c.groups[1].pages[s] if p >= 0]
    # the next position is 512 and sees keys from 443: pages 0..5 (positions < 384) are given back
    assert len(held) == 2 and c.groups[1].pages[s][:6] == [-1] * 6
    bt = c.block_table(1, [s, -1])
    assert bt.shape == (2, 8) and bt[0, 6] == held[0] and int(bt[1].abs().sum()) == 0
    c.free_slot(s)
    assert c.groups[1].pool.n_free == 10 and c.groups[0].pool.n_free == 10


def test_state_area_is_zero_for_a_new_slot():
    needs = [CacheNeed(kv=KVNeed(1, 8), state=StateNeed((3, 2)))]
    c = _cache(needs=needs, max_tokens=64 * 4, device="cpu", max_slots=3)
    assert c.states[0].shape == (3 + 1, 3, 2) and c.padding_slot == 3      # one more row, which no sequence owns
    s = c.alloc_slot()
    c.states[0][s] += 5.0
    c.free_slot(s)
    s2 = c.alloc_slot()
    assert s2 == s and float(c.states[0][s2].abs().sum()) == 0.0
    # an architecture without such a state has an empty area
    assert _cache(device="cpu").states == {}
    for _ in range(2):
        c.alloc_slot()
    with pytest.raises(CacheFull):
        c.alloc_slot()


def test_pages_of_a_step_that_did_not_run_go_back():
    c = _cache(max_tokens=64 * 6, device=None)
    a, b = c.alloc_slot(), c.alloc_slot()
    c.reserve([a, b], [70, 10])
    c.commit([a, b], [70, 10])
    free, va, vb = c.groups[0].pool.n_free, c.slot_version(a), c.slot_version(b)
    c.reserve([a, b], [60, 120])                   # a: 130 positions = one more page; b: 130 = two more
    assert c.groups[0].pool.n_free == free - 3 and c.slot_version(a) != va
    c.unreserve([a, b])                            # the step failed: nothing of it stays
    assert c.groups[0].pool.n_free == free and len(c.pages_of(0, a)) == 2 and len(c.pages_of(0, b)) == 1
    assert (c.length(a), c.length(b)) == (70, 10) and c.slot_version(b) != vb
    c.check()
    c.unreserve([a, b, 99])                        # nothing to give back, an unknown slot: no harm
    c.check()
    c.reserve([a], [1])                            # position 70 lies in a page the slot holds already
    assert c.groups[0].pool.n_free == free
