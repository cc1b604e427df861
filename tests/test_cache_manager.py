from __future__ import annotations

import random

import pytest

from kvcore_amd.cache.kv_manager import GroupConfig, KVManager
from kvcore_amd.cache.page_pool import PagePool, SlotPool


def test_pool_reserves_the_null_page_and_hands_out_in_order():
    """tests/test_kv_block_pool.py:57-75 (4 blocks: 3 free, ids 1,2,3; take 2 -> [1,2])."""
    pool = PagePool(4)
    assert pool.num_free == 3
    assert pool.take(2) == [1, 2]
    assert pool.num_free == 1
    pool.give_back([1, 2])
    assert pool.num_free == 3
    assert pool.take(3) == [3, 1, 2]  # first in, first out: freed pages queue behind free ones
    assert pool.usage() == 1.0
    pool.check()


def test_a_shuffled_pool_hands_out_every_page_once_in_another_order():
    plain_order = PagePool(40).take(39)
    shuffled = PagePool(40, shuffle_seed=1)
    order = shuffled.take(39)
    assert sorted(order) == plain_order == list(range(1, 40)) and order != plain_order
    assert PagePool(40, shuffle_seed=1).take(39) == order  # the seed fixes the order
    shuffled.check()


def test_pool_refuses_double_free_overdraw_and_foreign_ids():
    pool = PagePool(4)
    pages = pool.take(2)
    with pytest.raises(ValueError, match="only 1"):
        pool.take(2)
    pool.give_back(pages)
    with pytest.raises(RuntimeError, match="freed twice"):
        pool.give_back([pages[0]])
    with pytest.raises(ValueError, match="outside"):
        pool.give_back([9])
    pool.give_back([0])  # the null page is nobody's; giving it back is a no-op
    with pytest.raises(ValueError):
        PagePool(1)
    pool.check()


def test_slot_pool():
    slots = SlotPool(2)
    a, b = slots.take(), slots.take()
    assert {a, b} == {0, 1}
    with pytest.raises(ValueError):
        slots.take()
    slots.give_back(a)
    with pytest.raises(RuntimeError):
        slots.give_back(a)
    assert slots.take() == a


def make_manager(num_pages=8, page=2, seqs=4, window=0, max_len=64):
    return KVManager([GroupConfig(page, num_pages, window)], max_num_seqs=seqs, max_model_len=max_len)


def test_allocate_vector_of_the_reference():
    """tests/test_kv_manager.py:38-48: page size 2, 4 tokens, 8 blocks.  The reference has
    a list per layer ([1,2],[3,4]); a page here covers every layer, so one list [1,2]."""
    m = make_manager()
    m.admit("r")
    assert m.allocate("r", 0, 4) == [[1, 2]]
    assert m.page_ids("r") == [[1, 2]]
    assert m.num_free_pages() == [5]
    assert m.allocate("r", 4, 1) == [[3]]  # a fifth token starts a new page
    assert m.allocate("r", 5, 1) == [[]]   # the sixth fits
    with pytest.raises(ValueError):
        m.allocate("r", 6, 0)
    m.check()


def test_allocation_is_all_or_nothing_and_free_returns_tail_pages_first():
    m = make_manager(num_pages=6)  # 5 usable
    m.admit("a")
    m.admit("b")
    assert m.allocate("a", 0, 6) == [[1, 2, 3]]
    assert not m.can_fit("b", 6)
    assert m.allocate("b", 0, 6) is None
    assert m.num_free_pages() == [2] and m.page_ids("b") == [[]]
    assert m.allocate("b", 0, 4) == [[4, 5]]
    m.free("a")  # reverse order: 3, 2, 1 (single_type_kv_manager.py:177-182)
    assert m.allocate("b", 4, 6) == [[3, 2, 1]]
    m.free("b")
    assert m.num_free_pages() == [5]
    assert not m.is_admitted("a") and m.slots.num_free == 4
    m.check()


def test_request_cannot_outgrow_max_model_len_pages():
    m = make_manager(num_pages=40, max_len=8)
    m.admit("r")
    assert len(m.allocate("r", 0, 100)[0]) == 4  # kv_manager.py:455-478 clamps at max_model_len


def test_admission_needs_a_slot_and_a_fresh_id():
    m = make_manager(seqs=1)
    m.admit("a")
    with pytest.raises(ValueError, match="already"):
        m.admit("a")
    assert not m.has_free_slot()
    with pytest.raises(ValueError):
        m.admit("b")


def test_window_group_gives_pages_back_behind_the_window():
    m = make_manager(num_pages=8, page=4, window=6)
    m.admit("r")
    m.allocate("r", 0, 10)  # pages for tokens 0..9: 3 pages
    assert m.page_ids("r") == [[1, 2, 3]]
    # 10 tokens computed: the next query (position 10) needs keys 5..10 -> page 0 (0..3) is done
    assert m.release_behind_window("r", 10) == [1]
    assert m.page_ids("r") == [[0, 2, 3]] and m.num_free_pages() == [5]
    m.allocate("r", 10, 4)  # position 13: one more page; the freed one is behind the free ones
    assert m.page_ids("r") == [[0, 2, 3, 4]]
    assert m.release_behind_window("r", 14) == [2]  # next needs keys 9.. -> pages 0,1 done
    assert m.release_behind_window("r", 14) == [2]  # idempotent
    m.check()
    m.free("r")
    assert m.num_free_pages() == [7]
    m.check()


def test_two_groups_have_pages_of_their_own():
    m = KVManager([GroupConfig(4, 6, 0), GroupConfig(4, 4, 8)], max_num_seqs=2, max_model_len=64)
    m.admit("r")
    assert m.allocate("r", 0, 12) == [[1, 2, 3], [1, 2, 3]]
    assert m.allocate("r", 12, 4) is None  # the second pool is empty: nothing is taken from the first
    assert m.num_free_pages() == [2, 0]
    m.release_behind_window("r", 12)  # window 8: next needs keys 5.. -> page 0 done
    assert m.page_ids("r")[1] == [0, 2, 3]
    assert m.allocate("r", 12, 4) == [[4], [1]]
    m.check()


def test_groups_are_planned_for_the_same_number_of_tokens():
    from dataclasses import dataclass

    from kvcore_amd.cache.kv_manager import plan_groups

    @dataclass(frozen=True)
    class Need:
        page_size: int | None = None
        window: int = 0

    groups = plan_groups([Need(), Need(32, 0), Need(None, 64), Need(4, 0)], block_size=16, num_blocks=11)
    assert [(g.page_size, g.num_pages, g.window) for g in groups] == [
        (16, 11, 0), (32, 6, 0), (16, 11, 64), (4, 41, 0)]
    for g in groups:  # each holds the 160 tokens that ten blocks of sixteen hold
        assert (g.num_pages - 1) * g.page_size >= 160
    with pytest.raises(ValueError):
        plan_groups([Need()], 16, 1)


def test_pages_given_back_are_logged_when_asked_for():
    """The runner may poison pages that were given back; the manager says which they are."""
    m = KVManager([GroupConfig(4, 10, 0), GroupConfig(4, 10, 8)], max_num_seqs=2, max_model_len=64,
                  track_freed=True)
    m.admit("r")
    m.allocate("r", 0, 20)
    assert m.drain_freed() == [[], []]
    m.release_behind_window("r", 20)  # window 8: keys 13.. are needed, pages 0..2 go
    assert m.drain_freed() == [[], [1, 2, 3]]
    assert m.drain_freed() == [[], []]
    m.free("r")
    freed = m.drain_freed()
    assert sorted(freed[0]) == [1, 2, 3, 4, 5] and sorted(freed[1]) == [4, 5]
    quiet = make_manager()
    quiet.admit("q")
    quiet.allocate("q", 0, 4)
    quiet.free("q")
    assert quiet.drain_freed() == [[]]


@pytest.mark.parametrize("seed", range(5))
def test_no_page_is_lost_held_twice_or_freed_twice_under_random_traffic(seed):
    rng = random.Random(seed)
    window = rng.choice([0, 0, 12])
    m = KVManager([GroupConfig(4, 40, 0), GroupConfig(8, 24, window)], max_num_seqs=6, max_model_len=96)
    live: dict[str, int] = {}
    counter = 0
    for _ in range(600):
        action = rng.random()
        if action < 0.25 and m.has_free_slot():
            counter += 1
            rid = f"r{counter}"
            m.admit(rid)
            live[rid] = 0
        elif action < 0.85 and live:
            rid = rng.choice(list(live))
            n = rng.randint(1, 20)
            before = m.num_free_pages()
            got = m.allocate(rid, live[rid], n)
            if got is None:
                assert m.num_free_pages() == before  # nothing taken on failure
            else:
                live[rid] = min(live[rid] + n, 96)
                m.release_behind_window(rid, live[rid])
        elif live:
            rid = rng.choice(list(live))
            m.free(rid)
            del live[rid]
        m.check()
        assert sorted(m.live_requests()) == sorted(live)
    for rid in list(live):
        m.free(rid)
    m.check()
    assert m.num_free_pages() == [39, 23] and m.slots.num_free == 6
