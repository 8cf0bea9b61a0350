"""The cache manager alone: pages, block tables, groups with and without window, state slots."""
import random

import pytest

from lmsf_amd.cache import CacheError, CacheManager, GroupConfig, OutOfPages, PagePool, RELEASED


def test_pool_is_lifo_and_checks_holders():
    pool = PagePool(3)
    a, b = pool.allocate(), pool.allocate()
    assert (a, b) == (0, 1) and pool.num_free == 1
    pool.release(a)
    assert pool.allocate() == a                       # the page freed last is the next handed out
    with pytest.raises(CacheError, match="twice"):
        pool.release(2)                               # never handed out
    pool.release(b)
    with pytest.raises(CacheError, match="twice"):
        pool.release(b)
    with pytest.raises(CacheError, match="does not exist"):
        pool.release(7)
    pool.allocate(), pool.allocate()
    with pytest.raises(OutOfPages):
        pool.allocate()


def test_append_commit_and_tables():
    m = CacheManager([GroupConfig(page_size=4, num_pages=8)], num_state_slots=2)
    m.add_request("a")
    assert m.append("a", 6) == 0 and m.block_table("a", 0) == [0, 1]
    assert m.slot_mapping("a", 0, 0, 6) == [0, 1, 2, 3, 4, 5]
    with pytest.raises(CacheError, match="uncommitted"):
        m.append("a", 1)
    m.commit("a")
    assert m.num_tokens("a") == 6
    assert m.append("a", 2) == 6 and m.block_table("a", 0) == [0, 1]       # the last page had room for two
    m.commit("a")
    assert m.append("a", 1) == 8 and m.block_table("a", 0) == [0, 1, 2]    # position 8 opens a page
    m.commit("a")
    assert m.pages_needed("a", 3) == [0] and m.pages_needed("a", 4) == [1] and m.pages_needed(None, 9) == [3]
    m.add_request("b")
    m.append("b", 3)                                   # not committed: not yet in the pages
    assert m.tokens_held(["a", "nobody", "b", "a"]).tolist() == [9, 0, 0, 9] and m.tokens_held([]).tolist() == []
    m.commit("b")
    assert m.tokens_held(["b"]).tolist() == [3]
    m.check_invariants()


def test_out_of_pages_takes_nothing_and_rollback_returns_pages():
    m = CacheManager([GroupConfig(4, 3)], 2)
    m.add_request("a")
    m.append("a", 8)
    m.commit("a")
    m.add_request("b")
    with pytest.raises(OutOfPages):
        m.append("b", 5)
    assert m.num_free_pages() == 1 and m.block_table("b", 0) == []
    m.append("b", 4)
    assert m.num_free_pages() == 0
    m.rollback("b")
    assert m.num_free_pages() == 1 and m.num_tokens("b") == 0
    assert not m.can_append("a", 5) and m.can_append("a", 4) and not m.can_append("a", 4, reserve_pages=1)
    m.check_invariants()


def test_freeing_gives_back_everything_and_reuse_is_immediate():
    m = CacheManager([GroupConfig(2, 4)], 2)
    m.add_request("a")
    m.append("a", 5)
    m.commit("a")
    held = m.block_table("a", 0)
    m.free_request("a")
    assert m.num_free_pages() == 4 and not m.has_request("a")
    with pytest.raises(CacheError, match="holds no cache"):
        m.free_request("a")
    m.add_request("b")
    m.append("b", 2)
    assert m.block_table("b", 0) == [held[0]]          # the first page of the request that just ended
    m.check_invariants()


def test_state_slots():
    m = CacheManager([GroupConfig(4, 8)], num_state_slots=2)
    a, b = m.add_request("a"), m.add_request("b")
    assert {a.state_slot, b.state_slot} == {0, 1} and m.num_free_state_slots() == 0
    with pytest.raises(OutOfPages, match="state slots"):
        m.add_request("c")
    assert not m.can_append(None, 1) and m.can_append("a", 1)
    with pytest.raises(CacheError, match="already"):
        m.add_request("a")
    m.free_request("a")
    assert m.add_request("c").state_slot == a.state_slot
    m.check_invariants()


def test_window_group_gives_back_pages_the_window_has_passed():
    # two groups over the same requests: all keys, and a window of 6 with pages of 4
    m = CacheManager([GroupConfig(4, 16), GroupConfig(4, 4, window=6)], 2)
    m.add_request("a")
    m.append("a", 7)
    m.commit("a")                                      # next query at >= 7 reads keys > 1: page 0 still needed
    assert m.block_table("a", 1) == [0, 1]
    m.append("a", 3)
    m.commit("a")                                      # 10 tokens: keys >= 5 needed: block 0 (keys 0..3) passed
    assert m.block_table("a", 1) == [RELEASED, 1, 2] and m.num_free_pages(1) == 2
    assert m.block_table("a", 0) == [0, 1, 2]          # the full group keeps everything
    with pytest.raises(CacheError, match="given back"):
        m.slot_mapping("a", 1, 2, 1)
    for _ in range(30):                                # decoding on and on never needs more than 3 pages of the window group
        m.append("a", 1)
        m.commit("a")
        assert 4 - m.num_free_pages(1) <= 3
        m.check_invariants()
    m.free_request("a")
    assert m.num_free_pages(0) == 16 and m.num_free_pages(1) == 4
    m.check_invariants()


@pytest.mark.parametrize("seed", range(8))
def test_random_orders_lose_no_page(seed):
    rng = random.Random(seed)
    groups = [GroupConfig(rng.choice([1, 4, 16]), rng.randrange(6, 40)),
              GroupConfig(rng.choice([2, 8]), rng.randrange(6, 40), window=rng.choice([3, 10, 33]))]
    m = CacheManager(groups[:rng.choice([1, 2])], num_state_slots=5)
    live, next_id = {}, 0
    for _ in range(600):
        action = rng.random()
        if action < 0.25 and len(live) < 5:
            m.add_request(next_id)
            live[next_id] = 0
            next_id += 1
        elif action < 0.8 and live:
            rid = rng.choice(list(live))
            n = rng.choice([1, 1, 1, 2, 5, 17, 40])
            fits = m.can_append(rid, n)
            before = [m.num_free_pages(g) for g in range(len(m.groups))]
            try:
                start = m.append(rid, n)
            except OutOfPages:
                assert not fits
                assert before == [m.num_free_pages(g) for g in range(len(m.groups))]     # all or nothing
                continue
            assert fits and start == live[rid]
            for g in range(len(m.groups)):
                slots = m.slot_mapping(rid, g, start, n)
                assert len(set(slots)) == n
            if rng.random() < 0.15:
                m.rollback(rid)
            else:
                m.commit(rid)
                live[rid] += n
            assert m.num_tokens(rid) == live[rid]
        elif live:
            rid = rng.choice(list(live))
            m.free_request(rid)
            del live[rid]
        m.check_invariants()
        # slots of different live requests never collide
        for g, cfg in enumerate(m.groups):
            seen = set()
            for rid, n in live.items():
                lo = 0 if cfg.window is None else max(0, n - cfg.window + 1)
                if n > lo:
                    s = set(m.slot_mapping(rid, g, lo, n - lo))
                    assert not (s & seen)
                    seen |= s
    m.reset()
    assert all(m.num_free_pages(g) == m.groups[g].num_pages for g in range(len(m.groups)))
    assert m.num_free_state_slots() == 5
