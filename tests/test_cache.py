"""Cache bookkeeping: no slot or page lost, held twice or freed twice (no GPU; the store runs on CPU tensors)."""

import numpy as np
import pytest
import torch

from dryft_amd.cache import (CacheFull, CacheMisuse, CacheStore, KVNeed, PagePool, PageTable, SlotTable, StateNeed,
                             pages_for)


def test_page_pool_hands_out_each_page_once():
    pool = PagePool(5)
    a = pool.take(3)
    b = pool.take(2)
    assert sorted(a + b) == [0, 1, 2, 3, 4] and pool.free_count == 0
    with pytest.raises(CacheFull):
        pool.take(1)
    pool.give_back(a)
    assert pool.free_count == 3
    with pytest.raises(CacheMisuse):
        pool.give_back([a[0]])                      # freed twice
    with pytest.raises(CacheMisuse):
        pool.give_back([7])
    assert sorted(pool.take(3)) == sorted(a)        # used again


def test_slot_table():
    slots = SlotTable(3)
    held = [slots.acquire() for _ in range(3)]
    assert sorted(held) == [0, 1, 2]
    with pytest.raises(CacheFull):
        slots.acquire()
    slots.lengths[held[1]] = 40
    slots.release(held[1])
    with pytest.raises(CacheMisuse):
        slots.release(held[1])
    again = slots.acquire()
    assert again == held[1] and slots.lengths[again] == 0


def test_page_table_grows_by_need_and_releases_everything():
    table = PageTable(n_slots=2, n_pages=6, max_pages_per_slot=4)
    table.ensure(0, 1)
    table.ensure(0, 64)
    assert len(table.held_pages(0)) == 1
    table.ensure(0, 65)
    table.ensure(1, 130)
    assert len(table.held_pages(0)) == 2 and len(table.held_pages(1)) == 3 and table.pool.free_count == 1
    assert not set(table.held_pages(0)) & set(table.held_pages(1))
    with pytest.raises(CacheFull):
        table.ensure(0, 200)                        # two more pages, one free
    with pytest.raises(CacheFull):
        table.ensure(1, 4 * 64 + 1)                 # beyond a slot's table
    table.release(1)
    assert table.pool.free_count == 4 and (table.table[1] == -1).all()
    table.ensure(0, 256)
    assert table.pool.free_count == 2
    assert table.dirty == {0, 1}


def test_windowed_table_frees_pages_behind_the_window():
    table = PageTable(n_slots=1, n_pages=4, max_pages_per_slot=16, window=70)
    length = 0
    for _ in range(900):                            # far more tokens than four pages hold
        table.ensure(0, length + 1)
        length += 1
        table.trim(0, length)
        held = table.held_pages(0)
        assert len(held) <= 3 and len(set(held)) == len(held)
        first_needed = max(0, length - 70 + 1) // 64
        assert int(table.first[0]) <= first_needed   # every key the next token sees still has its page
    table.release(0)
    assert table.pool.free_count == 4


def make_store(**kw):
    needs = {0: KVNeed(2, 16), 1: KVNeed(2, 16), 2: KVNeed(1, 32), 3: StateNeed((3, 5)), 4: None,
             5: KVNeed(2, 16, window=100)}
    args = dict(max_tokens=640, n_slots=4, max_len=512, dtype=torch.float32, device="cpu")
    args.update(kw)
    return CacheStore(needs, **args)


def test_groups_have_storage_of_their_own():
    store = make_store()
    assert len(store.kv_groups) == 3 and len(store.state_groups) == 1
    shapes = sorted(tuple(g.k.shape) for g in store.kv_groups)
    assert shapes == [(1, 10, 1, 64, 32), (1, 10, 2, 64, 16), (2, 10, 2, 64, 16)]
    assert store.line(0).k.data_ptr() != store.line(1).k.data_ptr()
    assert store.line(0).page_table is store.line(1).page_table          # one group, one table
    assert store.line(0).page_table is not store.line(5).page_table      # the windowed group has its own
    assert store.line(5).window == 100 and store.line(0).window is None
    assert store.line(3).state.shape == (4, 3, 5) and store.line(4) is None
    assert store.bytes() == sum(2 * g.k.numel() * 4 for g in store.kv_groups) + 4 * 15 * 4


def test_steps_advance_lengths_and_release_resets(monkeypatch):
    store = make_store()
    slots = store.acquire(3)
    assert store.begin_step(slots, [5, 64, 100]) == [0, 0, 0]
    store.end_step(slots, [5, 64, 100])
    assert store.begin_step(slots[:2], [1, 1]) == [5, 64]
    store.end_step(slots[:2], [1, 1])
    assert [int(store.slots.lengths[s]) for s in slots] == [6, 65, 100]
    full = store.kv_groups[0]
    assert [len(full.table.held_pages(s)) for s in slots] == [1, 2, 2]
    assert (full.table_dev.numpy() == full.table.table).all()             # uploads keep the device copy in step
    store.line(3).state[slots[1]] = 7.0
    store.release([slots[1]])
    assert not store.line(3).state[slots[1]].any()                         # fixed-size state is zeroed
    assert int(store.slots.lengths[slots[1]]) == 0 and full.table.held_pages(slots[1]) == []
    with pytest.raises(CacheMisuse):
        store.release([slots[1]])
    with pytest.raises(CacheMisuse):
        store.begin_step([slots[1]], [1])                                  # a released slot cannot step
    with pytest.raises(CacheFull, match="longest sequence"):
        store.begin_step([slots[2]], [413])
    store.release([slots[0], slots[2]])
    for g in store.kv_groups:
        assert g.table.pool.free_count == g.table.pool.n_pages
    assert store.slots.free_count == 4


def test_token_budget_is_counted_in_whole_pages():
    store = make_store(max_tokens=256, n_slots=4)       # four pages
    slots = store.acquire(4)
    store.begin_step(slots, [1, 1, 1, 1])               # each sequence takes a whole page
    store.end_step(slots, [1, 1, 1, 1])
    store.begin_step(slots[:1], [63])                   # still within its first page
    store.end_step(slots[:1], [63])
    with pytest.raises(CacheFull):
        store.begin_step(slots[:1], [1])                # a fifth page does not exist
    store.release(slots[1:2])
    store.begin_step(slots[:1], [1])                    # ... until another sequence gives its page back
    store.end_step(slots[:1], [1])
    assert store.acquire(1) and store.slots.free_count == 0
    with pytest.raises(CacheFull):
        store.acquire(1)


def test_random_traffic_never_loses_or_doubles_anything():
    rng = np.random.default_rng(0)
    store = make_store(max_tokens=64 * 40, n_slots=6, max_len=1024)
    live: dict[int, int] = {}
    for _ in range(400):
        if live and rng.random() < 0.25:
            s = int(rng.choice(list(live)))
            store.release([s])
            del live[s]
        elif len(live) < 6 and rng.random() < 0.4:
            s = store.acquire(1)[0]
            assert s not in live
            live[s] = 0
        elif live:
            batch = [int(s) for s in rng.permutation(list(live))[: rng.integers(1, len(live) + 1)]]
            q = [int(rng.integers(1, 90)) for _ in batch]
            try:
                store.begin_step(batch, q)
            except CacheFull:
                continue
            store.end_step(batch, q)
            for s, n in zip(batch, q):
                live[s] += n
        for g in store.kv_groups:
            held = [p for s in range(6) for p in g.table.held_pages(s)]
            assert len(held) == len(set(held)), "a page is held twice"
            assert len(held) + g.table.pool.free_count == g.table.pool.n_pages, "a page was lost"
            for s, n in live.items():
                first, count = int(g.table.first[s]), int(g.table.count[s])
                assert count >= pages_for(n)
                if g.need.window is None:
                    assert first == 0
        assert store.slots.free_count + len(live) == 6
        assert all(int(store.slots.lengths[s]) == n for s, n in live.items())
    store.release(list(live))
    assert all(g.table.pool.free_count == g.table.pool.n_pages for g in store.kv_groups)
