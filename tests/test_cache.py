"""The cache's bookkeeping: no slot or page lost, held twice or freed twice (no GPU)."""
import random

import numpy as np

import pytest
import torch

from gpullama3_java_amd.cache import Cache, CacheFull, KVNeed, PagePool, SlotTable, StateNeed


def test_page_pool():
    pool = PagePool(5)
    a = pool.take(3)
    assert 0 not in a and len(set(a)) == 3 and pool.n_free == 1
    with pytest.raises(CacheFull):
        pool.take(2)
    assert pool.n_free == 1                                   # a refused request takes nothing
    pool.give_back(a[:2])
    with pytest.raises(RuntimeError):
        pool.give_back(a[:1])                                 # freed twice
    with pytest.raises(RuntimeError):
        pool.give_back([0])                                   # the sink page is never held
    assert pool.n_free == 3


def test_slot_table():
    st = SlotTable(3, 1)
    s = [st.take() for _ in range(3)]
    assert sorted(s) == [0, 1, 2]
    with pytest.raises(CacheFull):
        st.take()
    st.give_back(s[1])
    with pytest.raises(RuntimeError):
        st.give_back(s[1])
    assert st.take() == s[1]                                  # given back, used again


def make(max_tokens=640, max_context=256, n_slots=4, needs=None, state=None):
    needs = needs or [KVNeed(2, 16), KVNeed(2, 16), KVNeed(1, 32, window=8)]
    state = state or [None, StateNeed(6), None]
    return Cache(needs, state, max_tokens, max_context, n_slots, torch.float32, "cpu", page_size=64)


def test_groups_have_storage_of_their_own():
    c = make()
    assert len(c.groups) == 2
    assert c.groups[0].k.shape == (2, 11, 2, 64, 16) and c.groups[1].k.shape == (1, 11, 1, 64, 32)
    assert c.group_of == {0: (0, 0), 1: (0, 1), 2: (1, 0)}
    k, v = c.layer_kv(1)
    assert k.shape == (11, 2, 64, 16) and v.shape == (11, 2, 16, 64) and k.data_ptr() == c.groups[0].k[1].data_ptr()
    assert c.slot_state(1).shape == (5, 6) and c.slot_state(0) is None      # a row per slot and the sink row


def test_reserve_is_all_or_nothing():
    c = make()
    a, b = c.take_slot(), c.take_slot()
    c.reserve({a: 100, b: 10})
    c.advance(a, 100); c.advance(b, 10)
    third = c.take_slot()
    c.reserve({third: 200}); c.advance(third, 200)             # 4 of the 10 pages
    assert len(c.slots.pages[a][0]) == 2 and len(c.slots.pages[a][1]) == 2 and len(c.slots.pages[b][0]) == 1
    free = [g.pool.n_free for g in c.groups]
    with pytest.raises(CacheFull, match="longest"):
        c.reserve({a: 1, b: 300})                             # b would pass max_context
    with pytest.raises(CacheFull, match="pages"):
        c.reserve({a: 156, b: 246})                           # 2 + 3 more pages, 3 are free
    assert [g.pool.n_free for g in c.groups] == free and c.length(a) == 100
    c.reserve({a: 28})                                        # fits the pages already held
    assert [g.pool.n_free for g in c.groups] == free
    with pytest.raises(RuntimeError):
        c.reserve({3: 1})                                     # a slot nobody holds


def test_state_is_zeroed_when_a_slot_is_handed_out():
    c = make()
    s = c.take_slot()
    c.slot_state(1)[s] = 5.0
    c.give_back_slot(s)
    s2 = c.take_slot()
    assert s2 == s and torch.all(c.slot_state(1)[s2] == 0)


def test_random_traffic_keeps_the_books():
    rng = random.Random(0)
    c = make(max_tokens=64 * 12, max_context=300, n_slots=5)
    total_pages = [g.pool.n_pages - 1 for g in c.groups]
    live = {}
    for _ in range(2000):
        op = rng.random()
        if op < 0.3 and len(live) < 5:
            live[c.take_slot()] = 0
        elif op < 0.8 and live:
            s = rng.choice(list(live))
            n = rng.randint(1, 90)
            try:
                c.reserve({s: n})
                c.advance(s, n)
                live[s] += n
            except CacheFull:
                pass
        elif live:
            s = rng.choice(list(live))
            c.give_back_slot(s)
            del live[s]
            with pytest.raises(RuntimeError):
                c.give_back_slot(s)
        # the books: every page is free or held by exactly one live slot; lengths fit their pages
        for g, group in enumerate(c.groups):
            held = [p for s in live for p in c.slots.pages[s][g] if p]
            assert len(held) == len(set(held))
            assert len(held) + group.pool.n_free == total_pages[g]
            assert set(held) == group.pool._held
            for s, n in live.items():
                # a group without a window holds every page; with one, exactly the pages from the one
                # with the first key that the next token sees
                first = max(0, n + 1 - group.need.window) // 64 if group.need.window else 0
                assert [bool(p) for p in c.slots.pages[s][g]] == [i >= first for i in range(-(-n // 64))]
        for s, n in live.items():
            assert c.length(s) == n and all(len(c.slots.pages[s][g]) == -(-n // 64) for g in range(2))
        assert set(live) == c.slots.live and len(live) + len(c.slots._free) == 5
    for s in list(live):
        c.give_back_slot(s)
    assert all(g.pool.n_free == t for g, t in zip(c.groups, total_pages))


def test_a_slots_table_row_names_its_pages_then_the_sink():
    c = make()
    a = c.take_slot()
    c.reserve({a: 70})
    row = c.groups[0].table_host[a].tolist()
    assert row[:2] == c.slots.pages[a][0] and not any(row[2:])


def test_a_group_with_a_window_gives_back_the_pages_behind_it():
    c = make(max_tokens=64 * 8, max_context=400, n_slots=2, needs=[KVNeed(2, 16), KVNeed(1, 32, window=70)], state=[None, None])
    s = c.take_slot()
    full, windowed = c.groups[0].pool, c.groups[1].pool
    c.reserve({s: 130}); c.advance(s, 130)                      # the next token sees keys from 61 on: page 0 still
    assert full.n_free == 8 - 3 and windowed.n_free == 8 - 3
    c.reserve({s: 4}); c.advance(s, 4)                          # from 65 on: page 0 is out of reach
    assert c.slots.pages[s][1][0] == 0 and all(c.slots.pages[s][1][1:]) and windowed.n_free == 8 - 2
    assert all(c.slots.pages[s][0]) and full.n_free == 8 - 3    # the group without a window keeps everything
    c.reserve({s: 200}); c.advance(s, 200)                      # 334 tokens: from 265 on, pages 4 and 5 of 6
    assert [bool(p) for p in c.slots.pages[s][1]] == [False] * 4 + [True] * 2 and windowed.n_free == 8 - 2
    assert c.groups[1].table_host[s, :4].tolist() == [0, 0, 0, 0]    # the places of the pages given back point at the sink
    c.give_back_slot(s)
    assert full.n_free == 8 and windowed.n_free == 8


def test_the_table_of_every_group_follows_the_pages():
    """The host copy of each group's block table (a row per slot, the last row no sequence's) holds what
    the slots hold, and every change waits in ``dirty`` until it has travelled to the device."""
    c = Cache([KVNeed(2, 16), KVNeed(1, 32, window=100)], [None, None], 640, 640, 3, torch.float32, "cpu", page_size=64)
    a, b = c.take_slot(), c.take_slot()
    c.reserve({a: 200, b: 5}); c.advance(a, 200); c.advance(b, 5)
    W = c.max_pages_per_seq
    for g, group in enumerate(c.groups):
        assert group.table_host.shape == (4, W) and not group.table_host[c.sink_slot].any()
        for s in (a, b):
            pages = c.slots.pages[s][g]
            assert group.table_host[s, :len(pages)].tolist() == pages
        # after 200 tokens the first page of a lies behind the window of 100: its place names the sink page
        assert (group.table_host[a, 0] == 0) == (group.need.window is not None)
        assert {k: v for k, v in group.dirty.items()} == {
            s * W + i: int(group.table_host[s, i]) for s in (a, b) for i in range(len(c.slots.pages[s][g]))}
        group.dirty = {}
    c.reserve({a: 1}); c.advance(a, 1)                       # no new page: nothing to send
    assert all(not g.dirty for g in c.groups)
    c.reserve({b: 60}); c.advance(b, 60)                     # b's second page
    assert all(list(g.dirty) == [b * W + 1] for g in c.groups)


def test_sizes_that_the_tiles_do_not_fit_are_refused_when_the_cache_is_built():
    """Pages of a multiple of 32 positions and heads of a multiple of 16 elements: refused by name before
    any memory is taken, not by the first kernel launch."""
    def build(needs, **kw):
        return Cache(needs, [None] * len(needs), 256, 256, 2, torch.float32, "cpu", **kw)
    with pytest.raises(ValueError, match="head_dim 24"):
        build([KVNeed(2, 16), KVNeed(2, 24)])
    with pytest.raises(ValueError, match="v_head_dim 40"):
        build([KVNeed(2, 16, v_head_dim=40)])
    for page in (48, 16, 0, 70):
        with pytest.raises(ValueError, match="page_size"):
            build([KVNeed(2, 16)], page_size=page)
    assert build([KVNeed(2, 16)], page_size=96).page_size == 96
    build([KVNeed(2, 16, v_head_dim=40, values=False)])        # a size that is not stored is not checked


def test_values_of_another_size_or_none_at_all():
    """A need may ask for values of another head size than its keys, or for the first array alone (one
    vector per position); needs that differ in either form groups of their own."""
    c = Cache([KVNeed(2, 32), KVNeed(2, 32, v_head_dim=16), KVNeed(1, 48, values=False), KVNeed(2, 32)], [None] * 4,
              256, 256, 2, torch.float32, "cpu")
    assert len(c.groups) == 3 and c.group_of[0][0] == c.group_of[3][0]
    n_pages = 256 // 64 + 1
    k, v = c.layer_kv(0)
    assert k.shape == (n_pages, 2, 64, 32) and v.shape == (n_pages, 2, 32, 64)
    k, v = c.layer_kv(1)
    assert k.shape == (n_pages, 2, 64, 32) and v.shape == (n_pages, 2, 16, 64)
    k, v = c.layer_kv(2)
    assert k.shape == (n_pages, 1, 64, 48) and v is None
    s = c.take_slot()
    c.reserve({s: 100}); c.advance(s, 100)                     # every group hands out its own pages
    assert all(len(c.slots.pages[s][g]) == 2 for g in range(3))
    c.give_back_slot(s)
    assert all(g.pool.n_free == n_pages - 1 for g in c.groups)


def test_a_slot_that_is_taken_again_overwrites_its_rows_old_entries():
    """A slot's row of the block table keeps the page numbers of the sequence that held it before; the
    next sequence's pages overwrite them from the first place on, and every change is queued for the
    device."""
    c = Cache([KVNeed(2, 16)], [None], 640, 640, 2, torch.float32, "cpu")
    a = c.take_slot()
    c.reserve({a: 300}); c.advance(a, 300)
    old = list(c.slots.pages[a][0])
    other = c.take_slot()
    c.reserve({other: 64}); c.advance(other, 64)
    c.groups[0].dirty = {}
    c.give_back_slot(a)
    b = c.take_slot()
    assert b == a and c.length(b) == 0
    c.reserve({b: 70}); c.advance(b, 70)
    new = c.slots.pages[b][0]
    W = c.max_pages_per_seq
    assert len(new) == 2 and c.groups[0].table_host[b, :2].tolist() == new
    assert c.groups[0].dirty == {b * W + i: p for i, p in enumerate(new)}
    assert c.groups[0].table_host[b, 2:5].tolist() == old[2:5]         # stale, beyond the sequence's length: never read
    assert not c.groups[0].table_host[c.sink_slot].any()


def test_a_need_may_name_its_own_storage_type():
    c = Cache([KVNeed(2, 16), KVNeed(2, 16, dtype=torch.float64), KVNeed(2, 16)], [None] * 3, 256, 256, 2, torch.float32, "cpu")
    assert len(c.groups) == 2 and c.group_of == {0: (0, 0), 2: (0, 1), 1: (1, 0)}
    assert c.layer_kv(0)[0].dtype == torch.float32 and c.layer_kv(1)[0].dtype == torch.float64


def test_order_inside_a_page_host_functions_agree_with_the_formulas():
    """``cache/layout.py`` (reshapes) against the offset formulas written out as index arrays."""
    import torch
    import cache_order as O
    from gpullama3_java_amd.cache import layout as L
    for page, hs in ((64, 64), (32, 16), (96, 48), (64, 128)):
        k = np.arange(3 * page * hs, dtype=np.int64).reshape(3, page, hs)
        v = np.arange(3 * page * hs, dtype=np.int64).reshape(3, hs, page)
        assert np.array_equal(L.tile_keys(k), O.tile_keys(k)) and np.array_equal(L.tile_values(v), O.tile_values(v))
        assert np.array_equal(L.untile_keys(L.tile_keys(k)), k) and np.array_equal(L.untile_values(L.tile_values(v)), v)
        assert torch.equal(L.tile_keys(torch.as_tensor(k)), torch.as_tensor(O.tile_keys(k)))
        assert torch.equal(L.untile_values(torch.as_tensor(v)), O.untile_values(torch.as_tensor(v)))
        # a key row's 8 consecutive elements stay consecutive; 32 positions stay 32 * hs consecutive elements
        idx = O.key_index(page, hs)
        assert np.all(np.diff(idx.reshape(page, hs // 8, 8), axis=-1) == 1)
        assert all(set(idx[g * 32:(g + 1) * 32].ravel()) == set(range(g * 32 * hs, (g + 1) * 32 * hs)) for g in range(page // 32))
    with pytest.raises(ValueError, match="multiple"):
        L.tile_keys(np.zeros((48, 16)))
