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


# ---- the native manager against the plain one, operation by operation ------------------------------------
def _both(pages, window, slots, page_size=16):
    import plain_cache_manager as plain
    groups = [GroupSpec(None, (0,)), GroupSpec(window, (1, 2))]
    pgroups = [plain.GroupSpec(None, (0,)), plain.GroupSpec(window, (1, 2))]
    return CacheManager(groups, page_size, pages, slots), plain.CacheManager(pgroups, page_size, pages, slots)


def _same_state(m, p, live):
    assert m.free_pages() == p.free_pages() and m.free_slots() == p.free_slots()
    for g, (a, b) in enumerate(zip(m.pools, p.pools)):
        assert a._free == b._free, g                               # the same pages, to be handed out in the same order
    for rid in live:
        a, b = m.get(rid), p.get(rid)
        assert (a.length, a.reserved, a.tables, a.state_slot) == (b.length, b.reserved, b.tables, b.state_slot), rid
    assert sorted(m.live()) == sorted(p.live()) == sorted(live)


@pytest.mark.parametrize("seed", range(6))
def test_native_manager_follows_the_plain_one(seed):
    import plain_cache_manager as plain
    rng = random.Random(100 + seed)
    m, p = _both(pages=rng.choice([6, 10, 17]), window=rng.choice([24, 40, 7]), slots=4)
    live, next_id = [], 0
    for _ in range(500):
        op = rng.random()
        if op < 0.2:
            outcome = []
            for mgr, exc in ((m, OutOfSlots), (p, plain.OutOfSlots)):
                try:
                    outcome.append(mgr.add(next_id))
                except exc:
                    outcome.append("full")
            assert outcome[0] == outcome[1]
            if outcome[0] != "full":
                live.append(next_id)
            next_id += 1
        elif op < 0.8 and live:
            rid, n = rng.choice(live), rng.choice([1, 1, 1, 2, 5, 16, 31, 70])
            assert m.pages_needed(rid, n) == p.pages_needed(rid, n)
            needs = [(r, rng.choice([1, 3, 20])) for r in rng.sample(live, rng.randint(1, len(live)))]
            assert m.can_reserve(needs) == p.can_reserve(needs)
            outcome = []
            for mgr, exc in ((m, OutOfPages), (p, plain.OutOfPages)):
                try:
                    mgr.reserve(rid, n)
                    outcome.append("ok")
                except exc as e:
                    outcome.append((e.group, e.needed, e.free))
            assert outcome[0] == outcome[1]
            if outcome[0] == "ok":
                k = rng.choice([n, n, max(1, n // 2)])              # a step may commit less than was reserved
                m.commit(rid, k); p.commit(rid, k)
        elif live:
            rid = live.pop(rng.randrange(len(live)))
            m.free(rid); p.free(rid)
        m.check(); p.check()
        _same_state(m, p, live)
    for rid in live:
        with pytest.raises(ValueError, match="beyond"):
            m.commit(rid, 10 ** 6)
        with pytest.raises(ValueError, match="positive"):
            m.reserve(rid, 0)


def test_a_steps_arrays_from_the_native_manager():
    """Lengths, positions, block tables and write slots of a step, against the plain manager's tables."""
    import numpy as np
    m, p = _both(pages=40, window=24, slots=4)
    for mgr in (m, p):
        for rid, n in (("a", 37), ("b", 5), ("c", 70)):
            mgr.add(rid); mgr.reserve(rid, n); mgr.commit(rid, n)
        for rid, n in (("a", 3), ("b", 1), ("c", 20)):
            mgr.reserve(rid, n)
    rids, q_len = ["c", "a", "b"], [20, 3, 1]
    arr = m.step_arrays(rids, q_len, 8)
    start = [p.length(r) for r in rids]
    assert arr["start"].tolist() == start and arr["q_start"].tolist() == [0, 20, 23] and arr["kv_len"].tolist() == [90, 40, 6]
    assert arr["state_slots"].tolist() == [p.state_slot(r) for r in rids]
    assert arr["row_req"].tolist() == [0] * 20 + [1] * 3 + [2]
    assert arr["positions"].tolist() == list(range(70, 90)) + [37, 38, 39] + [5]
    for g in range(2):
        tables = [p.block_table(r, g) for r in rids]
        width = -(-max(len(t) for t in tables) // 8) * 8
        want = np.full((3, width), -1, dtype=np.int32)
        for i, t in enumerate(tables):
            want[i, :len(t)] = t
        assert np.array_equal(arr["block_tables"][g], want)
        slots = [tables[i][pos // 16] * 16 + pos % 16 for i, pos in zip(arr["row_req"].tolist(), arr["positions"].tolist())]
        assert arr["write_slots"][g].tolist() == slots
    with pytest.raises(RuntimeError, match="no page"):
        m.step_arrays(["b"], [40], 8)                                # 6 + 40 positions, pages for 6 + 1
    with pytest.raises(KeyError):
        m.step_arrays(["nobody"], [1], 8)
    empty = m.step_arrays([], [], 8)
    assert empty["positions"].shape == (0,) and [t.shape for t in empty["block_tables"]] == [(0, 8), (0, 8)]


def test_many_requests_in_one_call():
    m = two_groups(pages=12)
    for rid, n in (("a", 20), ("b", 3)):
        m.add(rid); m.reserve(rid, n); m.commit(rid, n)
    snap = m.snapshot(["a", "b"])
    assert m.unchanged(snap, ["a", "b"]) and not m.unchanged(snap, ["b", "a"]) and not m.unchanged(snap, ["a"])
    m.reserve("a", 1); m.reserve("b", 1)
    assert m.unchanged(snap, ["a", "b"])                       # pages taken ahead move nothing
    m.commit_each(["a", "b"], 1)
    assert (m.length("a"), m.length("b")) == (21, 4) and not m.unchanged(snap, ["a", "b"])
    with pytest.raises(ValueError, match="beyond"):
        m.commit_each(["a", "b"], 1)                           # nothing reserved: neither moves
    assert (m.length("a"), m.length("b")) == (21, 4)
    snap = m.snapshot(["a", "b"])
    m.free("b"); m.add("b"); m.reserve("b", 4); m.commit("b", 4)
    assert not m.unchanged(snap, ["a", "b"])                   # the same name and length, another request
    m.check()
