"""The cache manager's bookkeeping: addressing and pool discipline of the reference
(`inferrs-models/src/kv_cache.rs:80-222`), all-or-nothing reservation, groups of layers with
pages of their own, windows that give pages back, state slots; and that under random orders of
requests no page is lost, held twice or freed twice."""
import random

import pytest

from inferrs_amd.cache import RELEASED, CacheError, CacheManager, PagePool, SlotPool
from inferrs_amd.parts.base import FixedState, PagedKV

FULL = PagedKV(2, 16)
WINDOW = PagedKV(2, 16, window=10)


def test_pool_is_fifo_and_counts_references():
    pool = PagePool(4)
    assert pool.allocate(3) == [0, 1, 2]
    assert pool.allocate(2) is None and pool.num_free == 1          # all or nothing
    pool.free([1])
    assert pool.allocate(2) == [3, 1]                               # front of the list, freed pages at the back
    with pytest.raises(CacheError, match="freed twice"):
        pool.free([1, 1])
    with pytest.raises(CacheError, match="does not belong"):
        pool.free([9])


def test_slot_addressing_follows_the_reference():
    # kv_cache.rs:183-192: slot = table[pos / bs] * bs + pos % bs
    m = CacheManager({0: FULL}, page_size=4, num_pages=8, max_seqs=2)
    m.add_sequence("a")
    m.sequences["a"].tables[0] = [5, 2]
    assert m.slot_ids("a", 0, 2, 5) == [5 * 4 + 2, 5 * 4 + 3, 2 * 4 + 0, 2 * 4 + 1, 2 * 4 + 2]


def test_reserve_is_all_or_nothing_and_commit_advances():
    m = CacheManager({0: FULL, 1: FULL}, page_size=4, num_pages=3, max_seqs=2)
    m.add_sequence("a")
    assert m.reserve("a", 9)                       # 3 pages
    assert m.sequences["a"].reserved == 9 and m.groups[0].pool.num_free == 0
    m.add_sequence("b")
    assert not m.reserve("b", 1) and m.sequences["b"].tables[0] == []
    m.commit("a", 9)
    assert m.sequences["a"].length == 9 and m.sequences["a"].reserved == 0
    assert m.reserve("a", 3) and not m.reserve("a", 1)      # the 12th token still fits the third page
    with pytest.raises(CacheError, match="commit"):
        m.commit("a", 4)
    m.free_sequence("a")
    assert m.groups[0].pool.num_free == 3
    with pytest.raises(CacheError, match="not live"):
        m.free_sequence("a")
    m.check_invariants()


def test_layers_with_the_same_needs_share_a_group():
    needs = {0: FULL, 1: WINDOW, 2: FULL, 3: FixedState((8,)), 4: None, 5: WINDOW}
    m = CacheManager(needs, page_size=4, num_pages=[6, 4], max_seqs=3)
    assert [(g.need, g.layers) for g in m.groups] == [(FULL, [0, 2]), (WINDOW, [1, 5])]
    assert [s.layer for s in m.states] == [3]
    assert m.layer_group == {0: 0, 2: 0, 1: 1, 5: 1}
    with pytest.raises(CacheError, match="page counts"):
        CacheManager(needs, page_size=4, num_pages=[6], max_seqs=3)


def test_a_window_gives_pages_back_once_it_has_passed_them():
    m = CacheManager({0: FULL, 1: WINDOW}, page_size=4, num_pages=[8, 4], max_seqs=1)
    m.add_sequence("a")
    for step in range(20):                         # one token at a time; the window group never needs > 4 pages
        assert m.reserve("a", 1), step
        m.commit("a", 1)
        m.check_invariants()
    seq = m.sequences["a"]
    # the next query is at position 20 and reads keys 11..20: pages 0 and 1 (keys 0..7) are gone
    assert seq.tables[1][:2] == [RELEASED, RELEASED] and RELEASED not in seq.tables[1][2:]
    assert RELEASED not in seq.tables[0] and len(seq.tables[0]) == 5
    with pytest.raises(CacheError, match="released"):
        m.slot_ids("a", 1, 7, 1)
    m.free_sequence("a")
    assert [g.pool.num_free for g in m.groups] == [8, 4]


def test_state_slots_lowest_free_first():
    m = CacheManager({0: FixedState((4,))}, page_size=4, num_pages=0, max_seqs=3)
    assert [m.add_sequence(i).state_slot for i in "abc"] == [0, 1, 2]
    with pytest.raises(CacheError, match="slots are in use"):
        m.add_sequence("d")
    m.free_sequence("b")
    assert m.add_sequence("d").state_slot == 1
    pool = SlotPool(1)
    pool.allocate()
    with pytest.raises(CacheError):
        pool.free(1)


@pytest.mark.parametrize("seed", range(8))
def test_random_orders_of_requests_keep_every_page_accounted_for(seed):
    rng = random.Random(seed)
    m = CacheManager({0: FULL, 1: WINDOW, 2: FULL}, page_size=rng.choice([1, 3, 4, 16]),
                     num_pages=[rng.randint(4, 40), rng.randint(4, 40)], max_seqs=5)
    live, next_id = [], 0
    for _ in range(1500):
        roll = rng.random()
        if roll < 0.15 and len(live) < 5:
            m.add_sequence(next_id)
            live.append(next_id)
            next_id += 1
        elif roll < 0.3 and live:
            m.free_sequence(live.pop(rng.randrange(len(live))))
        elif live:
            sid = rng.choice(live)
            n = rng.choice([1, 1, 1, 2, 7, 33])
            before = [g.pool.num_free for g in m.groups], [list(t) for t in m.sequences[sid].tables.values()]
            if m.reserve(sid, n):
                m.commit(sid, rng.randint(0, n)) if rng.random() < 0.2 else m.commit(sid, n)
                if m.sequences[sid].reserved:                    # a partial commit: the rest comes later
                    m.commit(sid, m.sequences[sid].reserved)
            else:                                               # a refusal takes nothing
                assert before == ([g.pool.num_free for g in m.groups], [list(t) for t in m.sequences[sid].tables.values()])
        m.check_invariants()
    for sid in live:
        m.free_sequence(sid)
    m.check_invariants()
    assert all(g.pool.num_free == g.pool.num_pages for g in m.groups) and m.slots.num_free == 5


def test_state_arrays_count_in_the_pool_sizing():
    """When the pool is sized from free memory, the fixed-size state of every request slot is paid first."""
    import torch
    from inferrs_amd.cache import CacheManager, CacheStorage
    from inferrs_amd.parts import FixedState, PagedKV
    manager = CacheManager({0: PagedKV(2, 16), 1: FixedState((1000,), torch.float32), 2: PagedKV(2, 16, None, 24)}, 8, 0, 5)
    assert CacheStorage.state_bytes(manager) == 5 * 1000 * 4
    assert CacheStorage.page_bytes(manager, torch.bfloat16) == (2 * 8 * 32 + 2 * 8 * 40) * 2


def test_paged_needs_with_one_array_or_values_as_rows():
    """What a paged need may ask of the storage beside keys and transposed values: no value array at all, or values as
    rows; needs that differ in this do not share a group, and a page's bytes follow."""
    keys_only = PagedKV(1, 24, values=False)
    rows = PagedKV(2, 16, None, 8, value_layout="rows")
    assert keys_only.value_dim == 0 and keys_only.page_elements(4) == 24 * 4
    assert rows.page_elements(4) == 2 * 4 * (16 + 8)
    manager = CacheManager({0: PagedKV(2, 16), 1: keys_only, 2: rows, 3: PagedKV(2, 16, None, 8)}, 4, 6, 2)
    assert len(manager.groups) == 4
    with pytest.raises(ValueError, match="value_layout"):
        PagedKV(2, 16, value_layout="sideways")
