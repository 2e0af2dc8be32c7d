"""The cache's book-keeping: no slot or page lost, held twice or freed twice."""
import random

import pytest
import torch

from trapetum_amd.cache import CacheError, FreeList, ModelCache, StateSpec, TokenSpec


def make(max_tokens=512, max_context=256, max_slots=4, page=16, window=40):
    kv = lambda w: TokenSpec.of(w, k=(2, 16), v=(2, 16))
    specs = [kv(window), kv(None), kv(window), StateSpec((3, 5)), None]
    return ModelCache(specs, max_tokens, max_context, max_slots, page, torch.float32, torch.device("cpu"))


def test_free_list():
    f = FreeList(3, "thing")
    assert [f.take(), f.take(), f.take()] == [0, 1, 2]
    with pytest.raises(CacheError, match="no free thing"):
        f.take()
    f.give_back(1)
    with pytest.raises(CacheError, match="twice"):
        f.give_back(1)
    with pytest.raises(CacheError, match="does not exist"):
        f.give_back(7)
    assert f.take() == 1 and f.held() == [0, 1, 2]


def test_groups_and_sites():
    c = make()
    assert len(c.token_groups) == 2 and len(c.state_groups) == 1
    local, glob = c.token_groups
    assert local.entries == [0, 2] and glob.entries == [1]
    assert local.pages.rows_cap == 48 and glob.pages.rows_cap is None        # window 40 -> ring of 3 pages of 16
    # 4 slots with rings of 3 pages never hold more than 12 pages; the other group may hold all 32; one spare each
    assert tuple(local.pools["k"].shape) == (2, 12 + 1, 2, 16, 16) and tuple(glob.pools["v"].shape) == (1, 32 + 1, 2, 16, 16)
    assert local.spare_page == 12 and glob.spare_page == 32 and c.spare_slot == 4
    assert c.site(0).group_index == 0 and c.site(2).index_in_group == 1 and c.site(4) is None
    assert tuple(c.site(3).state.shape) == (4 + 1, 3, 5)                      # one spare slot
    t = c.page_table(0, [c.spare_slot], width=3)                              # the spare slot's row names the spare page
    assert list(t[0]) == [12, -1, -1]
    wide = make(window=1000)                                                  # a window beyond the context keeps every row
    assert wide.token_groups[0].pages.rows_cap is None


def test_pages_follow_lengths():
    c = make()
    s = c.acquire()
    c.grow(s, 17)
    assert [len(g.pages.lists[s]) for g in c.token_groups] == [2, 2]
    c.grow(s, 100)                                                            # 117 tokens: ring stays at 3 pages
    assert [len(g.pages.lists[s]) for g in c.token_groups] == [3, 8]
    assert c.tokens_held() == 128 and c.length(s) == 117
    t = c.page_table(0, [s], width=5)
    assert t.shape == (1, 5) and list(t[0, 3:]) == [-1, -1] and sorted(t[0, :3]) == sorted(c.token_groups[0].pages.lists[s])
    with pytest.raises(CacheError, match="context overflow"):
        c.grow(s, 200)
    c.release(s)
    assert c.tokens_held() == 0 and [g.pages.pool.available() for g in c.token_groups] == [12, 32]
    with pytest.raises(CacheError, match="twice"):
        c.release(s)


def test_full_cache_is_refused_without_damage():
    c = make(max_tokens=64)                                                   # 4 pages per group
    a, b = c.acquire(), c.acquire()
    c.grow(a, 40)
    with pytest.raises(CacheError, match="full"):
        c.check_grow([a, b], [1, 30])
    assert c.length(a) == 40 and c.length(b) == 0
    c.check_grow([a, b], [1, 16])
    with pytest.raises(CacheError, match="twice"):
        c.check_grow([a, a], [1, 1])
    with pytest.raises(CacheError, match="not in use"):
        c.check_grow([3], [1])


def test_state_is_zeroed_when_a_slot_is_taken():
    c = make()
    s = c.acquire()
    c.site(3).state[s] += 5.0
    c.release(s)
    assert c.acquire() == s and float(c.site(3).state[s].abs().sum()) == 0.0


def test_random_walk_never_loses_a_page():
    rng = random.Random(0)
    c = make(max_tokens=1024, max_context=200, max_slots=6)
    live = {}
    for _ in range(2000):
        op = rng.random()
        if op < 0.3 and len(live) < 6:
            live[c.acquire()] = 0
        elif op < 0.8 and live:
            s = rng.choice(list(live))
            n = rng.randint(1, 30)
            try:
                c.check_grow([s], [n])
            except CacheError:
                continue
            c.grow(s, n)
            live[s] += n
        elif live:
            s = rng.choice(list(live))
            c.release(s)
            del live[s]
        assert c.live_slots() == sorted(live)
        for g in c.token_groups:
            owned = [p for s in live for p in g.pages.lists.get(s, [])]
            assert len(owned) == len(set(owned))                              # no page held twice
            assert len(owned) + g.pages.pool.available() == g.pages.pool.n   # none lost
            assert sorted(owned) == g.pages.pool.held()
            for s, n in live.items():
                assert len(g.pages.lists.get(s, [])) == g.pages.pages_needed(n)
    for s in list(live):
        c.release(s)
    assert all(g.pages.pool.available() == g.pages.pool.n for g in c.token_groups)
    assert c.book.slots.available() == 6
