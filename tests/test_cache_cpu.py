"""The cache manager's bookkeeping: no page lost, held twice or freed twice (no GPU)."""

import random

import pytest

from kestrel_amd.cache import CacheManager, OutOfPages, PagePool
from kestrel_amd.parts.specs import CacheSpec, StateSpec

FULL = CacheSpec(2, 16, None)
WINDOW = CacheSpec(2, 16, 24)


def _manager(needs=None, page_size=4, n_pages=16, max_requests=4):
    needs = needs or [(FULL, None, None), (FULL, None, None)]
    return CacheManager(needs, page_size, n_pages, max_requests)


def test_pool_refuses_double_free():
    pool = PagePool(4)
    pages = pool.take(2)
    pool.give_back(pages)
    with pytest.raises(AssertionError, match="freed twice"):
        pool.give_back(pages[:1])
    with pytest.raises(OutOfPages):
        pool.take(5)


def test_growth_block_table_and_slot_mapping():
    m = _manager()
    a = m.admit()
    m.ensure(a, 9)                                # 3 pages of 4
    assert len(m.block_table(0, a)) == 3 and m.length(a) == 9
    table = m.block_table(0, a)
    assert m.slot_of_position(0, a, 6) == table[1] * 4 + 2      # slot = page * page_size + offset
    m.ensure(a, 9)
    m.ensure(a, 5)                                # never shrinks
    assert len(m.block_table(0, a)) == 3
    m.ensure(a, 17)
    assert len(m.block_table(0, a)) == 5
    m.check()
    m.release(a)
    assert m.groups[0].pool.free_count == 16
    with pytest.raises(AssertionError, match="released twice"):
        m.release(a)


def test_freed_pages_are_used_again_last_freed_first():
    m = _manager()
    a = m.admit()
    m.ensure(a, 8)
    pages_a = list(m.block_table(0, a))
    m.release(a)
    b = m.admit()
    m.ensure(b, 8)
    assert m.block_table(0, b) == pages_a          # the same physical pages, in the same order
    m.check()


def test_out_of_pages_changes_nothing():
    m = _manager(n_pages=4)
    a, b = m.admit(), m.admit()
    m.ensure(a, 12)
    with pytest.raises(OutOfPages, match="Cannot reserve"):
        m.ensure(b, 8)
    assert m.block_table(0, b) == [] and m.length(b) == 0
    m.ensure(b, 4)
    m.check()


def test_promises_at_admission():
    m = _manager(n_pages=8)
    a = m.admit(reserve_length=20)                 # 5 pages promised
    assert m.pages_available(0) == 3
    assert m.can_admit(12) and not m.can_admit(13)
    with pytest.raises(OutOfPages):
        m.admit(reserve_length=16)
    b = m.admit(reserve_length=12)
    m.ensure(b, 12)
    m.ensure(a, 20)                                 # cannot fail: it was promised
    m.check()
    m.release(a)
    assert m.pages_available(0) == 5
    m.release(b)
    m.check()
    assert m.pages_available(0) == 8


def test_slots_run_out():
    m = _manager(max_requests=2)
    m.admit(), m.admit()
    assert not m.can_admit(1)
    with pytest.raises(OutOfPages, match="slot"):
        m.admit()


def test_groups_have_pools_of_their_own_and_windows_give_pages_back():
    needs = [(FULL, None, None), (WINDOW, None, None), (FULL, None, None), (WINDOW, None, 1)]
    m = _manager(needs, page_size=4, n_pages=32)
    assert len(m.groups) == 2 and m.groups[0].entries == [0, 2] and m.groups[1].entries == [1]
    caches = m.layer_caches()
    assert [c.group for c in caches] == [0, 1, 0, 1] and [c.writes for c in caches] == [True, True, True, False]
    a = m.admit()
    held = []
    for length in range(1, 101):
        m.ensure(a, length)
        m.trim(a, length)
        m.check()
        held.append(sum(1 for p in m.block_table(1, a) if p >= 0))
        # every key the next query may read is still backed
        for pos in range(m.window_start(1, length), length):
            m.slot_of_position(1, a, pos)
    assert max(held) <= m.pages_for(1, 100, portion=1)
    assert sum(1 for p in m.block_table(0, a) if p >= 0) == 25   # the full group keeps everything
    assert m.groups[1].pool.free_count >= 32 - 7
    m.release(a)
    m.check()
    assert all(g.pool.free_count == 32 for g in m.groups)


def test_reading_a_cache_with_other_needs_is_refused():
    with pytest.raises(ValueError, match="cannot read the cache"):
        CacheManager([(FULL, None, None), (WINDOW, None, 0)], 4, 8, 2)


def test_state_slots_without_a_gpu_are_bookkeeping_only():
    m = CacheManager([(None, StateSpec((3, 5)), None)], 4, 8, 3)
    assert m.groups == [] and m.layer_caches()[0].group is None
    a = m.admit()
    m.ensure(a, 100)                                # no groups: nothing to back
    m.release(a)
    m.check()


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_of_requests(seed):
    rng = random.Random(seed)
    needs = [(FULL, None, None), (WINDOW, None, None)] if seed % 2 else [(FULL, None, None)]
    m = _manager(needs, page_size=4, n_pages=24, max_requests=5)
    live = {}
    for _ in range(600):
        action = rng.random()
        if action < 0.25 and m.free_slots:
            reserve = rng.choice([0, 0, rng.randint(1, 40)])
            try:
                slot = m.admit(reserve)
                live[slot] = 0
            except OutOfPages:
                pass
        elif action < 0.8 and live:
            slot = rng.choice(list(live))
            target = live[slot] + rng.randint(1, 9)
            try:
                m.ensure(slot, target)
                live[slot] = target
                m.trim(slot, target)
            except OutOfPages:
                pass
        elif live:
            slot = rng.choice(list(live))
            m.release(slot)
            del live[slot]
        m.check()
    for slot in list(live):
        m.release(slot)
    m.check()
    assert all(g.pool.free_count == 24 and g.pool.promised_unheld == 0 for g in m.groups)
