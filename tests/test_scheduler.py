"""The scheduler's decisions (no GPU): a fake step stands in for the model, as the reference's
tests use a mock backend that records its inputs (tests/unit/test_unified_batching.cpp:26-53) and
one that checks positions (tests/unit/test_scheduler.cpp:2680-2760)."""
import pytest

from inferflux_amd.cache import CacheManager, GroupSpec
from inferflux_amd.engine.scheduler import RequestRefused, Scheduler, SchedulerConfig


def make(pages=64, page_size=16, slots=8, max_position=4096, groups=None, **cfg):
    """(Portions are ``chunked_prefill_tokens`` long with or without decoding requests beside them unless a test says
    ``prefill_tokens_alone``.)"""
    m = CacheManager(groups or [GroupSpec(None, (0,))], page_size, pages, slots)
    cfg.setdefault("prefill_tokens_alone", cfg.get("chunked_prefill_tokens", 512))
    return m, Scheduler(m, SchedulerConfig(**cfg), max_position)


def fake_token(context):
    """A deterministic 'model': the next token is a function of everything before it."""
    h = 17
    for t in context:
        h = (h * 31 + t + 1) % 1009
    return h % 97


def drive(m, s, max_steps=10000, log=None):
    """The engine's loop without a GPU.  Checks what every step must satisfy and returns each
    request's generated tokens."""
    seqs = {q.rid: q for q in list(s.waiting)}
    cached = {}                                        # rid -> the tokens the 'cache' holds
    steps = 0
    while s.has_work():
        plan = s.schedule()
        assert plan.items, "work left but nothing planned"
        assert plan.n_tokens <= s.config.max_batch_tokens
        assert len(plan.items) <= s.config.max_batch_size and len({i.seq.rid for i in plan.items}) == len(plan.items)
        for rid in plan.preempted:
            cached.pop(rid, None)
        for it in plan.items:
            assert m.length(it.seq.rid) == len(cached.get(it.seq.rid, [])) == it.seq.computed   # positions are consistent
            assert len(it.tokens) <= s.config.largest_portion
            m.reserve(it.seq.rid, len(it.tokens)); m.commit(it.seq.rid, len(it.tokens))       # what runner.step does
            cached.setdefault(it.seq.rid, []).extend(it.tokens)
            s.advance(it)
        m.check()
        if log is not None:
            log.append([(i.seq.rid, len(i.tokens), i.wants_logits) for i in plan.items])
        for it in plan.items:
            if it.wants_logits:
                it.seq.generated.append(fake_token(cached[it.seq.rid]))
                if len(it.seq.generated) >= it.seq.max_new:
                    cached.pop(it.seq.rid)
                    s.finish(it.seq)
        steps += 1
        assert steps < max_steps
    return {rid: q.generated for rid, q in seqs.items()}


def expected(prompt, n):
    ctx, out = list(prompt), []
    for _ in range(n):
        out.append(fake_token(ctx)); ctx.append(out[-1])
    return out


def test_a_long_prompt_is_cut_into_portions_with_logits_on_the_last():
    # the reference's own case: 1200 tokens -> 512, 512, 176, then decode steps (test_unified_batching.cpp:316-420)
    m, s = make(pages=128)
    s.add("a", list(range(1200)), 4)
    log = []
    out = drive(m, s, log=log)
    assert log == [[("a", 512, False)], [("a", 512, False)], [("a", 176, True)], [("a", 1, True)], [("a", 1, True)], [("a", 1, True)]]
    assert out["a"] == expected(range(1200), 4)
    assert m.free_pages() == [128] and not m.live()


def test_portions_are_long_while_nobody_decodes():
    """By default a prompt goes in portions of 2,048 while no request decodes (nobody waits for it), and of
    chunked_prefill_tokens as soon as one does."""
    m = CacheManager([GroupSpec(None, (0,))], 16, 1024, 8)
    s = Scheduler(m, SchedulerConfig(), 8192)
    assert (s.config.chunked_prefill_tokens, s.config.portion_alone, s.config.largest_portion) == (512, 2048, 2048)
    s.add("a", list(range(5000)), 3)
    s.add("b", list(range(100)), 40)
    log = []
    drive(m, s, log=log)
    # a alone at first (b joins in the same step: both are prompts), then b decodes beside a's shorter portions
    assert log[0] == [("a", 2048, False), ("b", 100, True)]
    assert log[1] == [("a", 512, False), ("b", 1, True)] and log[2] == [("a", 512, False), ("b", 1, True)]
    assert SchedulerConfig(chunked_prefill_tokens=4096).portion_alone == 4096
    assert SchedulerConfig(chunked_prefill_tokens=64, prefill_tokens_alone=64).largest_portion == 64


def test_decodes_first_then_the_budget_goes_to_prompts():
    m, s = make(pages=256, max_batch_tokens=100, chunked_prefill_tokens=64)
    s.add("a", list(range(10)), 50)
    s.add("b", list(range(150)), 5)
    s.add("c", list(range(30)), 5)
    log = []
    drive(m, s, log=log)
    assert log[0] == [("a", 10, True), ("b", 64, False), ("c", 26, False)]     # 100 tokens exactly
    assert log[1] == [("a", 1, True), ("b", 64, False), ("c", 4, True)]
    assert log[2] == [("a", 1, True), ("b", 22, True), ("c", 1, True)]
    assert all(sum(n for _, n, _ in step) <= 100 for step in log)


def test_every_running_request_advances_and_order_is_first_come_first_served():
    m, s = make(pages=256, max_batch_size=2)
    for i, n in enumerate((5, 6, 7)):
        s.add(i, list(range(n)), 3)
    log = []
    out = drive(m, s, log=log)
    assert [r for r, _, _ in log[0]] == [0, 1]                # only two places: request 2 waits
    first_2 = next(i for i, st in enumerate(log) if any(r == 2 for r, _, _ in st))
    assert first_2 == 3                                        # it joins the step after request 0 and 1 finish
    for i, n in enumerate((5, 6, 7)):
        assert out[i] == expected(range(n), 3)


def test_pages_run_out_the_youngest_is_preempted_and_results_do_not_change():
    # 8 pages of 16: three requests of 40+40 tokens need 15 pages in the end -> somebody has to wait
    m, s = make(pages=8)
    prompts = {i: [i * 7 + k for k in range(40)] for i in range(3)}
    for i, p in prompts.items():
        s.add(i, p, 40)
    log = []
    out = drive(m, s, log=log)
    for i, p in prompts.items():
        assert out[i] == expected(p, 40), i                   # recomputation changes nothing
    assert m.free_pages() == [8] and not m.live()
    # the oldest request is never the victim
    m2, s2 = make(pages=8)
    seqs = [s2.add(i, p, 40) for i, p in prompts.items()]
    drive(m2, s2)
    assert seqs[0].preemptions == 0 and sum(q.preemptions for q in seqs) >= 1


def test_preempted_request_returns_to_the_front_with_its_tokens_as_prompt():
    m, s = make(pages=4, page_size=16)
    a = s.add("a", list(range(30)), 30)
    b = s.add("b", list(range(100, 120)), 30)
    plan = s.schedule()
    assert [i.seq.rid for i in plan.items] == ["a", "b"] and m.free_pages() == [0]
    for it in plan.items:
        m.commit(it.seq.rid, len(it.tokens)); s.advance(it); it.seq.generated.append(1)
    s.schedule()                                               # a: 31 tokens fit its 2 pages; b: 21 fit
    for q in (a, b):
        m.commit(q.rid, 1); q.computed += 1; q.generated.append(2)
    a.computed, b.computed = 31, 21
    # make a need a third page: fast-forward it to the page edge
    m.reserve("a", 1); m.commit("a", 1); a.computed += 1; a.generated.append(3)     # 32 tokens in cache
    plan = s.schedule()                                        # a needs page 3 -> b (younger) is preempted
    assert plan.preempted == ["b"] and [i.seq.rid for i in plan.items] == ["a"]
    assert s.waiting[0] is b and b.prompt == list(range(100, 120)) + [1, 2] and b.computed == 0 and b.folded == 2
    assert not m.has("b")


def test_refusals():
    m, s = make(pages=4, max_position=100)
    with pytest.raises(RequestRefused, match="context overflow"):
        s.add("a", list(range(90)), 11)
    with pytest.raises(RequestRefused, match="never fit"):
        s.add("b", list(range(60)), 10)                        # 70 tokens = 5 pages > 4
    with pytest.raises(RequestRefused, match="empty"):
        s.add("c", [], 5)
    s.add("d", [1, 2], 5)
    with pytest.raises(RequestRefused, match="already"):
        s.add("d", [1], 5)


def test_windowed_group_lets_long_requests_through_a_small_pool():
    groups = [GroupSpec(None, (0,)), GroupSpec(32, (1,))]
    m = CacheManager(groups, 16, [64, 8], 4)
    s = Scheduler(m, SchedulerConfig(chunked_prefill_tokens=48, prefill_tokens_alone=48), 2048)
    s.add("a", list(range(500)), 100)
    out = drive(m, s)
    assert out["a"] == expected(range(500), 100)
    assert m.free_pages() == [64, 8]
    # with portions of up to 2,048 tokens while nobody decodes (the default) the window's pool of 8 pages cannot take
    # a portion, and the request is refused when it is added, not when it is half-way
    s = Scheduler(m, SchedulerConfig(chunked_prefill_tokens=48), 2048)
    with pytest.raises(RequestRefused, match="can never fit"):
        s.add("b", list(range(500)), 100)


@pytest.mark.parametrize("seed", range(4))
def test_random_workloads_finish_with_the_right_tokens(seed):
    import random
    rng = random.Random(seed)
    m, s = make(pages=rng.choice([10, 16, 40]), slots=4, max_batch_size=4, max_batch_tokens=rng.choice([24, 64, 512]),
                chunked_prefill_tokens=rng.choice([8, 32, 512]))
    prompts = {i: [rng.randrange(500) for _ in range(rng.choice([1, 5, 17, 40, 70]))] for i in range(9)}
    news = {i: rng.choice([1, 2, 20, 50]) for i in prompts}
    for i, p in prompts.items():
        s.add(i, p, news[i])
    out = drive(m, s)
    for i, p in prompts.items():
        assert out[i] == expected(p, news[i])
    assert m.free_pages() == [m.pools[0].num_pages]


def test_priority_decides_admission_and_the_default_is_first_come_first_served():
    # one place in the batch: the order of admission is the order of service
    m, s = make(pages=64, max_batch_size=1)
    s.add("low", [1, 2, 3], 2)
    s.add("high", [4, 5, 6], 2, priority=5)
    s.add("mid", [7, 8], 2, priority=2)
    s.add("high2", [9], 2, priority=5)
    log = []
    drive(m, s, log=log)
    order = []
    for step in log:
        for rid, _, _ in step:
            if rid not in order:
                order.append(rid)
    assert order == ["high", "high2", "mid", "low"]            # by priority, arrival among equals


def test_the_score_hook_is_the_references_priority_plus_age():
    # scheduler/batch_selection_policy.cpp:10-20: every 2 s of waiting count as one step of priority
    from inferflux_amd.engine.scheduler import priority_age_score
    now = [0.0]
    m = CacheManager([GroupSpec(None, (0,))], 16, 64, 8)
    s = Scheduler(m, SchedulerConfig(max_batch_size=1), 4096, score=priority_age_score(2000.0), clock=lambda: now[0])
    old = s.add("old", [1, 2], 1)                               # priority 0, arrives at t = 0
    now[0] = 3.0
    new = s.add("new", [3, 4], 1, priority=1)                   # priority 1, arrives at t = 3
    assert s.score(old, 3.0) == 1.5 and s.score(new, 3.0) == 1.0
    plan = s.schedule()                                         # at t = 3 the old request has aged past the new one
    assert [i.seq.rid for i in plan.items] == ["old"]
    m2 = CacheManager([GroupSpec(None, (0,))], 16, 64, 8)
    s2 = Scheduler(m2, SchedulerConfig(max_batch_size=1), 4096, score=priority_age_score(2000.0), clock=lambda: now[0])
    now[0] = 0.0
    s2.add("old", [1, 2], 1)
    now[0] = 1.0
    s2.add("new", [3, 4], 1, priority=1)
    assert [i.seq.rid for i in s2.schedule().items] == ["new"]  # one second of age does not outweigh a priority step


def test_a_stream_of_more_important_arrivals_does_not_starve_a_waiting_request():
    """One place in the batch, a request of priority 0 waiting, and a request of priority 1 arriving every half
    second: under the default score the old request's age outgrows the newcomers' priority after two seconds and it
    is admitted; under the priority alone it waits as long as the stream lasts."""
    from inferflux_amd.engine.scheduler import priority_score

    def admitted_after(score):
        now = [0.0]
        m = CacheManager([GroupSpec(None, (0,))], 16, 64, 8)
        s = Scheduler(m, SchedulerConfig(max_batch_size=1), 4096, score=score, clock=lambda: now[0])
        s.add("first", [1, 2], 1, priority=1)
        s.add("patient", [3, 4], 1)
        for tick in range(1, 41):
            plan = s.schedule()
            assert len(plan.items) == 1
            if plan.items[0].seq.rid == "patient":
                return tick
            it = plan.items[0]
            m.commit(it.seq.rid, len(it.tokens)); s.advance(it); s.finish(it.seq)     # a request takes one step
            now[0] += 0.5
            s.add(f"vip{tick}", [5, 6], 1, priority=1)
        return None

    assert admitted_after(None) is not None and admitted_after(None) <= 8       # about 2 s / 0.5 s, and a few ticks
    assert admitted_after(priority_score) is None


def test_the_victim_is_the_lowest_priority_then_the_youngest():
    m, s = make(pages=4, page_size=16)
    a = s.add("a", list(range(30)), 30)                         # oldest, priority 0
    b = s.add("b", list(range(100, 120)), 30, priority=3)       # younger but more important
    plan = s.schedule()
    assert [i.seq.rid for i in plan.items] == ["b", "a"] and m.free_pages() == [0]
    for it in plan.items:
        m.commit(it.seq.rid, len(it.tokens)); s.advance(it); it.seq.generated.append(1)
    # b reaches its page edge (32 tokens) and needs a third page: a, of lower priority, has to go although it is older
    for _ in range(12):
        m.reserve("b", 1); m.commit("b", 1); b.computed += 1; b.generated.append(2)
    plan = s.schedule()
    assert plan.preempted == ["a"] and [i.seq.rid for i in plan.items] == ["b"]
    assert s.waiting[0] is a and not m.has("a")


def test_a_victims_tokens_return_to_the_steps_budget():
    """A running request of low priority is planned, then a more important one needs a page and takes the first
    one's: the token the victim had been charged is free again for an admission in the same step."""
    m, s = make(pages=3, page_size=16, max_batch_tokens=2)
    a = s.add("a", list(range(16)), 30)                         # priority 0, admitted first
    s.config.max_batch_tokens = 64
    plan = s.schedule()
    for it in plan.items:
        m.commit("a", len(it.tokens)); s.advance(it); a.generated.append(1)
    b = s.add("b", list(range(100, 116)), 30, priority=5)
    plan = s.schedule()                                         # a decodes (its 17th token: a second page), b is admitted
    assert [(i.seq.rid, len(i.tokens)) for i in plan.items] == [("a", 1), ("b", 16)] and m.free_pages() == [0]
    for it in plan.items:
        m.commit(it.seq.rid, len(it.tokens)); s.advance(it); it.seq.generated.append(2)
    s.add("c", [7, 8, 9, 10, 11], 4, priority=1)
    s.config.max_batch_tokens = 2
    plan = s.schedule()
    # a was dealt its token, then b needed a page for its 17th and a, of lower priority, had to go; the token a had
    # been charged went to c, which outranks the preempted a in the queue
    assert plan.preempted == ["a"]
    assert [(i.seq.rid, len(i.tokens)) for i in plan.items] == [("b", 1), ("c", 1)] and plan.n_tokens == 2
    assert s.waiting[0] is a
