"""The cache's books: no slot or page lost, held twice or given back twice; lengths, groups,
windows and per-sequence state."""
import random

import pytest
import torch

from libllm_amd import CacheError
from libllm_amd.cache import PAGE, PagePool, SequenceCache, SlotTable, pages_for
from libllm_amd.parts import CacheNeed, Plane, StateNeed, rows_plane
from libllm_amd.parts.kv_pages import kv_need


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
    # two attention layers of one shape, one with a window and another shape, a mixer that keeps
    # one latent row a token in a type of its own, and a layer that caches nothing
    latent = CacheNeed("full", (rows_plane("z", (5,), PAGE, torch.float64),))
    needs = [kv_need(2, 16, 0, PAGE), kv_need(2, 16, 0, PAGE), kv_need(1, 32, 100, PAGE), latent, None]
    states = [None, StateNeed((3,)), None, StateNeed((2, 2)), None]
    cache = SequenceCache(needs, states, max_tokens=64 * 12, max_position=640, dtype=torch.float32, device="cpu")
    assert [g.entries for g in cache.groups] == [[0, 1], [2], [3]]
    # keys in blocks of 16 dims, values in halves of 32 positions (parts/kv_pages.py)
    g0, g1, g2 = cache.groups
    assert g0.planes["k"].shape == (2, 13, 2, 1, PAGE, 16) and g0.planes["v"].shape == (2, 13, 2, 2, 16, 32)
    assert g1.planes["k"].shape == (1, 13, 1, 2, PAGE, 16) and g1.planes["v"].shape == (1, 13, 1, 2, 32, 32)
    assert list(g2.planes) == ["z"] and g2.planes["z"].shape == (1, 13, PAGE, 5) and g2.planes["z"].dtype == torch.float64
    view = cache.kv_view(3)
    assert view.plane("z").shape == (13, PAGE, 5) and view.need.plane("z").layout == "rows" and view.need.plane("k") is None
    with pytest.raises(KeyError, match="no plane 'k'"):
        view.plane("k")
    assert cache.kv_view(4) is None
    assert cache.state[1].shape == (13, 3) and cache.state[3].shape == (13, 2, 2) and 0 not in cache.state
    with pytest.raises(CacheError, match="twice"):
        SequenceCache([CacheNeed("full", (Plane("a", (PAGE, 2)), Plane("a", (PAGE, 3))))], [None], max_tokens=64,
                      max_position=64, dtype=torch.float32, device="cpu")
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
        full, win, lat = cache.groups
        for rid, slot in live.items():
            n = cache.length(slot)
            assert sorted(full.held.get(slot, {})) == list(range(pages_for(n))) == sorted(lat.held.get(slot, {}))
            if n:
                first = max(0, n + 1 - 100) // PAGE       # pages wholly behind the window are given back
                assert sorted(win.held.get(slot, {})) == list(range(first, pages_for(n)))
    for rid in list(live):
        cache.release(rid)
    cache.check()
    assert all(g.pool.n_free == g.pool.n_pages for g in cache.groups) and cache.slots.n_free == cache.slots.n_slots


def test_reused_slot_starts_clean_and_tables_follow():
    cache = SequenceCache([kv_need(1, 16, 0, PAGE)], [StateNeed((4,))], max_tokens=256, max_position=256,
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
    from libllm_amd.parts import kv_pages as layout
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
