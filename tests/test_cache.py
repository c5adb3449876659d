"""The cache's books: no slot or page lost, held twice or given back twice; lengths, groups,
windows and per-sequence state."""
import random

import pytest
import torch

from libllm_amd import CacheError
from libllm_amd.cache import PAGE, PagePool, SequenceCache, SlotTable, pages_for
from libllm_amd.parts import CacheNeed, StateNeed


def test_page_pool():
    pool = PagePool(5)
    a = pool.take(2)
    b = pool.take(3)
    assert sorted(a + b) == [0, 1, 2, 3, 4] and pool.n_free == 0
    with pytest.raises(CacheError):
        pool.take(1)
    pool.give_back(a)
    with pytest.raises(CacheError):
        pool.give_back(a)                                   # given back twice
    with pytest.raises(CacheError):
        pool.give_back([b[0], b[0]])                        # twice in one call: nothing changes
    assert pool.n_free == 2
    with pytest.raises(CacheError):
        pool.give_back([7])
    assert pool.take(2) == sorted(a)                        # lowest first: reuse is deterministic
    pool.check()


def test_slot_table():
    t = SlotTable(2)
    assert t.acquire("a") == 0 and t.acquire("b") == 1
    with pytest.raises(CacheError):
        t.acquire("a")                                      # held twice
    with pytest.raises(CacheError):
        t.acquire("c")                                      # none free
    assert t.release("a") == 0
    with pytest.raises(CacheError):
        t.release("a")                                      # freed twice
    assert t.acquire("c") == 0 and t.slot_of("c") == 0 and not t.holds("a")
    t.check()


def test_random_traffic_keeps_the_books():
    rnd = random.Random(1)
    needs = [CacheNeed("full", 2, 16), CacheNeed("full", 2, 16), CacheNeed("window", 1, 32, 100), None]
    states = [None, StateNeed((3,)), None, StateNeed((2, 2))]
    cache = SequenceCache(needs, states, max_tokens=64 * 12, max_position=640, dtype=torch.float32, device="cpu")
    assert len(cache.groups) == 2 and cache.groups[0].entries == [0, 1] and cache.groups[1].entries == [2]
    # keys in blocks of 16 dims, values in halves of 32 positions (cache/layout.py)
    assert cache.groups[0].k.shape == (2, 13, 2, 1, PAGE, 16) and cache.groups[0].v.shape == (2, 13, 2, 2, 16, 32)
    assert cache.groups[1].k.shape == (1, 13, 1, 2, PAGE, 16) and cache.groups[1].v.shape == (1, 13, 1, 2, 32, 32)
    assert cache.state[1].shape == (13, 3) and cache.state[3].shape == (13, 2, 2) and 0 not in cache.state
    live = {}
    for step in range(400):
        op = rnd.random()
        if op < 0.3 and len(live) < 6:
            rid = "r%d" % step
            slot = cache.admit(rid)
            live[rid] = slot
        elif op < 0.8 and live:
            rid = rnd.choice(list(live))
            n = rnd.choice([1, 1, 1, 5, 70])
            slot = live[rid]
            try:
                cache.reserve(slot, n)
            except CacheError:
                cache.check()                                # a refusal changes nothing
                continue
            before = cache.length(slot)
            cache.state[1][slot] += 1
            cache.commit(slot, n)
            assert cache.length(slot) == before + n
        elif live:
            rid = rnd.choice(list(live))
            cache.release(rid)
            del live[rid]
        cache.check()
        full, win = cache.groups
        for rid, slot in live.items():
            n = cache.length(slot)
            assert sorted(full.held.get(slot, {})) == list(range(pages_for(n)))
            if n:
                first = max(0, n + 1 - 100) // PAGE       # pages wholly behind the window are given back
                assert sorted(win.held.get(slot, {})) == list(range(first, pages_for(n)))
    for rid in list(live):
        cache.release(rid)
    cache.check()
    assert all(g.pool.n_free == g.pool.n_pages for g in cache.groups) and cache.slots.n_free == cache.slots.n_slots


def test_reused_slot_starts_clean_and_tables_follow():
    cache = SequenceCache([CacheNeed("full", 1, 16)], [StateNeed((4,))], max_tokens=256, max_position=256,
                          dtype=torch.float32, device="cpu")
    s = cache.admit("a")
    cache.reserve(s, 100)
    cache.commit(s, 100)
    cache.state[0][s] = 7.0
    cache.flush()
    g = cache.groups[0]
    assert g.table[s, :2].tolist() == [0, 1] and g.table[s, 2].item() == g.sink_page
    cache.release("a")
    cache.flush()
    assert (g.table[s] == g.sink_page).all()
    s2 = cache.admit("b")
    assert s2 == s and cache.length(s2) == 0 and (cache.state[0][s2] == 0).all()
    with pytest.raises(CacheError):
        cache.reserve(s2, 257)                              # beyond max_position
    with pytest.raises(CacheError):
        cache.release("a")
    t = cache.admit("c")
    cache.reserve(t, 200)
    with pytest.raises(CacheError):
        cache.reserve(s2, 65)                               # 4 pages exist, 4 held after this would be 6
    cache.check()
    assert cache.tokens_held() == 256


def test_page_layout_round_trip():
    """Keys and values written through the layout's helpers come back; a head size that is no
    multiple of 16 pads its last block of dims; the flat offsets are the kernels' formulas."""
    from libllm_amd.cache import layout
    for hd in (16, 24, 64, 80):
        k = torch.zeros(layout.key_pages_shape(3, 2, hd))
        v = torch.zeros(layout.value_pages_shape(3, 2, hd))
        assert k.shape == (3, 2, (hd + 15) // 16, 64, 16) and v.shape == (3, 2, 2, hd, 32)
        g = torch.Generator().manual_seed(hd)
        keys, vals = torch.randn((5, 2, hd), generator=g), torch.randn((5, 2, hd), generator=g)
        pages, offs = torch.tensor([0, 2, 2, 1, 0]), torch.tensor([0, 63, 31, 32, 17])
        layout.write_keys(k, pages, offs, keys)
        layout.write_values(v, pages, offs, vals)
        assert torch.equal(layout.read_keys(k, pages, offs, hd), keys)
        assert torch.equal(layout.read_values(v, pages, offs), vals)
        kb, vb = k.shape[2] * 16 * 64, hd * 64                 # elements per (page, kv head)
        for i in range(5):
            for head in range(2):
                for d in (0, 7, hd - 1):
                    page, pos = int(pages[i]), int(offs[i])
                    at = (page * 2 + head) * kb + (d // 16) * 1024 + pos * 16 + d % 16
                    assert k.reshape(-1)[at] == keys[i, head, d]
                    at = (page * 2 + head) * vb + (pos // 32) * hd * 32 + d * 32 + pos % 32
                    assert v.reshape(-1)[at] == vals[i, head, d]
