"""The cache manager's accounting (no GPU): no page lost, held twice or freed twice."""
import random

import pytest

from inferflux_amd.cache import CacheManager, GroupSpec, OutOfPages, OutOfSlots, PagePool


def two_groups(pages=12, window=40, page_size=16, slots=4):
    return CacheManager([GroupSpec(None, (0,)), GroupSpec(window, (1, 2))], page_size, pages, slots)


def test_pool_reuses_most_recently_freed_and_rejects_double_free():
    p = PagePool(3)
    a, b = p.take(), p.take()
    assert (a, b) == (0, 1) and p.num_free == 1
    p.release(a)
    assert p.take() == a
    p.release(b)
    with pytest.raises(ValueError, match="freed twice"):
        p.release(b)
    p.retain(a)
    p.release(a)
    assert p.refs(a) == 1 and p.num_free == 2
    p.release(a)
    assert p.num_free == 3


def test_pages_follow_lengths_and_return_on_free():
    m = two_groups()
    m.add("a")
    m.reserve("a", 17)
    assert m.pages_needed("a", 17) == [0, 0] and [len(t) for t in m.get("a").tables] == [2, 2]
    m.commit("a", 17)
    assert m.length("a") == 17 and m.pages_needed("a", 15) == [0, 0] and m.pages_needed("a", 16) == [1, 1]
    assert m.slot_of("a", 0, 16) == m.block_table("a", 0)[1] * 16
    m.check()
    m.free("a")
    assert m.free_pages() == [12, 12]
    with pytest.raises(KeyError, match="freed twice"):
        m.free("a")
    m.check()


def test_reserve_is_all_or_nothing():
    m = two_groups(pages=3)
    m.add("a"); m.add("b")
    m.reserve("a", 32); m.commit("a", 32)
    before = (m.free_pages(), [list(t) for t in m.get("b").tables])
    with pytest.raises(OutOfPages) as ei:
        m.reserve("b", 33)
    assert ei.value.needed == 3 and ei.value.free == 1
    assert (m.free_pages(), [list(t) for t in m.get("b").tables]) == before
    assert not m.can_reserve([("b", 17)]) and m.can_reserve([("b", 16)])
    assert not m.can_reserve([("a", 16), ("b", 16)])
    m.check()


def test_window_group_gives_pages_back_as_the_window_passes():
    m = two_groups(pages=12, window=40)
    m.add("a")
    n = 0
    for step in (30, 30, 1, 1, 50, 7):
        m.reserve("a", step); m.commit("a", step); n += step
        m.check()
        full, win = m.get("a").tables
        assert all(p >= 0 for p in full) and len(full) == -(-n // 16)
        first_needed = n - 40 + 1                       # oldest position the next query may read
        for b, p in enumerate(win):
            dead = (b + 1) * 16 <= first_needed         # every position of the block lies before it
            assert (p < 0) == dead, (n, b, p)
    held = sum(1 for p in m.get("a").tables[1] if p >= 0)
    assert held <= 40 // 16 + 2
    with pytest.raises(ValueError, match="released"):
        m.slot_of("a", 1, 0)
    m.free("a")
    assert m.free_pages() == [12, 12]


def test_state_slots():
    m = two_groups(slots=2)
    s = {m.add("a"), m.add("b")}
    assert s == {0, 1}
    with pytest.raises(OutOfSlots):
        m.add("c")
    with pytest.raises(ValueError, match="already live"):
        m.add("a")
    m.free("a")
    assert m.add("c") in (0, 1) and m.state_slot("c") != m.state_slot("b")
    m.check()


@pytest.mark.parametrize("seed", range(5))
def test_random_orders_never_lose_or_double_book_a_page(seed):
    rng = random.Random(seed)
    m = two_groups(pages=10, window=24, slots=4)
    lengths = {}
    next_id = 0
    for _ in range(600):
        op = rng.random()
        if op < 0.25 and len(lengths) < 4:
            m.add(next_id); lengths[next_id] = 0; next_id += 1
        elif op < 0.85 and lengths:
            rid = rng.choice(list(lengths))
            n = rng.choice([1, 1, 1, 2, 5, 16, 31])
            try:
                m.reserve(rid, n)
                m.commit(rid, n)
                lengths[rid] += n
            except OutOfPages:
                victim = max(lengths, key=lengths.get)
                m.free(victim); del lengths[victim]
        elif lengths:
            rid = rng.choice(list(lengths))
            m.free(rid); del lengths[rid]
        m.check()
        for rid, n in lengths.items():
            assert m.length(rid) == n
            assert sum(1 for p in m.block_table(rid, 0) if p >= 0) == -(-n // 16)
    for rid in list(lengths):
        m.free(rid)
    m.check()
    assert m.free_pages() == [10, 10]
