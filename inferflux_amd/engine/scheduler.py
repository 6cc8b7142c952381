"""Continuous batching with chunked prefill under a token budget.  No GPU needed: the scheduler
decides, the engine executes.

Every step the running set is formed anew: each running request that is decoding contributes one
token, the rest of the budget is dealt to prompts as portions of at most
``chunked_prefill_tokens`` (of ``prefill_tokens_alone``, 2,048 by default, in a step in which nobody
decodes and so nobody waits for the prompts), and waiting requests are admitted first come first served while a
place in the batch, budget and pages for their first portion are there.  Only the last portion
of a prompt asks for logits.

Option names and defaults are the reference's (scheduler/scheduler.h:64-89): max_batch_size 32,
max_batch_tokens 16384, chunked_prefill_tokens 512.  What differs, by design: the reference
charges a prompt its whole length against the budget and skips what does not fit
(scheduler/scheduler.cpp:327-378, 2039-2049), reserves ceil(prompt/16)+1 blocks at admission
(2327-2335) and has no answer to pages running out during decoding, because its sequence slots
have a fixed extent (runtime/backends/cuda/inferflux_cuda_executor.cpp:3240-3253).  Here pages are
taken as tokens arrive, and when a running request needs a page and none is free the most
recently admitted running request is preempted: its pages are given back and it returns to the
front of the waiting queue with prompt + generated tokens as its new prompt (recomputation).
A request that could never fit the pool alone, or whose prompt + max_tokens exceeds the model's
positions, is refused when it is added (the reference: context_overflow, scheduler.cpp:2303-2324).

Order of admission.  The reference sorts its queues by a score, priority + age_ms / 2000, ties by
arrival (scheduler/batch_selection_policy.cpp:10-20; scheduler/scheduler.cpp:2013-2031).  Here a
request carries a ``priority`` (0 unless given) and the scheduler a ``score`` function of the
waiting request; the waiting request with the highest score is admitted next, the earlier arrival
among equals.  The default score is the reference's (``priority_age_score``): every two seconds
of waiting count as one step of priority, so a steady stream of more important arrivals cannot
keep a waiting request out for ever, and while nobody sets a priority the order is first come
first served; ``priority_score`` is the priority alone.  The best-scoring request that does
not fit blocks those behind it (no overtaking by smaller requests).  When pages run out the
victim is the running request of lowest priority, the most recently admitted among those.
"""
from __future__ import annotations

import collections
import dataclasses
import time
from typing import Callable, Deque, Hashable, List, Optional, Sequence

from ..cache.manager import CacheManager, OutOfPages


@dataclasses.dataclass
class SchedulerConfig:
    max_batch_size: int = 32           # requests in a step (the reference caps this at 64)
    max_batch_tokens: int = 16384      # tokens in a step
    chunked_prefill_tokens: int = 512  # largest portion of a prompt in a step beside requests that are decoding
    # Largest portion in a step in which nobody decodes (None: the larger of chunked_prefill_tokens and 2,048).  Portions are
    # short so that decoding requests do not wait long for a prompt; while there are none, nobody waits, and the matrix
    # products of 2,048 rows run at 0.43 of the chip's peak where those of 512 run at 0.27.
    prefill_tokens_alone: Optional[int] = None

    PREFILL_ALONE = 2048

    def validate(self) -> None:
        if self.max_batch_size < 1 or self.max_batch_tokens < 1 or self.chunked_prefill_tokens < 1:
            raise ValueError("scheduler limits must be positive")
        if self.prefill_tokens_alone is not None and self.prefill_tokens_alone < 1:
            raise ValueError("prefill_tokens_alone must be positive (or None)")

    @property
    def portion_alone(self) -> int:
        return self.prefill_tokens_alone if self.prefill_tokens_alone is not None else max(self.chunked_prefill_tokens, self.PREFILL_ALONE)

    @property
    def largest_portion(self) -> int:
        return max(self.chunked_prefill_tokens, self.portion_alone)


class RequestRefused(ValueError):
    pass


@dataclasses.dataclass(eq=False)     # requests are compared by identity (they sit in lists and deques)
class Sequence_:
    """A request as the scheduler sees it.

    The cache has to hold ``prompt`` and then every generated token but the newest, which is
    the input of the next decode step.  ``computed`` counts the tokens that are in the cache.
    After a preemption the tokens generated so far are appended to ``prompt`` (``folded`` of
    them are) and everything is computed again.
    """
    rid: Hashable
    prompt: List[int]
    max_new: int
    generated: List[int] = dataclasses.field(default_factory=list)
    computed: int = 0
    arrival: int = 0
    admitted_at: int = -1              # admission order; -1 while waiting
    preemptions: int = 0
    n_prompt_original: int = 0
    folded: int = 0
    priority: int = 0                  # higher is admitted earlier and preempted later
    arrival_time: float = 0.0          # the scheduler's clock when the request was added

    @property
    def is_prefilling(self) -> bool:
        return self.computed < len(self.prompt)


@dataclasses.dataclass
class PlannedItem:
    seq: Sequence_
    tokens: List[int]
    wants_logits: bool


@dataclasses.dataclass
class StepPlan:
    items: List[PlannedItem]
    preempted: List[Hashable]
    admitted: List[Hashable]

    @property
    def n_tokens(self) -> int:
        return sum(len(i.tokens) for i in self.items)


def priority_score(seq: "Sequence_", now: float) -> float:
    """The request's priority alone; equal priorities are served in arrival order.  Under it a stream of more
    important arrivals keeps a less important request waiting for as long as it lasts."""
    return float(seq.priority)


def priority_age_score(aging_divisor_ms: float = 2000.0) -> Callable[["Sequence_", float], float]:
    """The default, and the reference's policy: every ``aging_divisor_ms`` of waiting adds one to the effective
    priority (scheduler/batch_selection_policy.cpp:10-20)."""
    def score(seq: "Sequence_", now: float) -> float:
        return float(seq.priority) + (now - seq.arrival_time) * 1e3 / aging_divisor_ms
    return score


class Scheduler:
    def __init__(self, manager: CacheManager, config: SchedulerConfig, max_position: int,
                 score: Optional[Callable[["Sequence_", float], float]] = None,
                 clock: Callable[[], float] = time.monotonic):
        """``score(request, now)``: the waiting request with the highest is admitted next (``priority_age_score()``
        unless given); ``clock`` gives ``now`` and the requests' arrival times, in seconds."""
        config.validate()
        self.manager, self.config, self.max_position = manager, config, max_position
        self.score, self.clock = score or priority_age_score(), clock
        self.waiting: Deque[Sequence_] = collections.deque()
        self.running: List[Sequence_] = []
        self._arrivals = 0
        self._admissions = 0

    # ---- requests -----------------------------------------------------------------
    def add(self, rid: Hashable, prompt: Sequence[int], max_new: int, priority: int = 0) -> Sequence_:
        prompt = [int(t) for t in prompt]
        if not prompt:
            raise RequestRefused(f"request {rid!r}: empty prompt")
        if any(s.rid == rid for s in list(self.waiting) + self.running):
            raise RequestRefused(f"request {rid!r} is already queued or running")
        total = len(prompt) + max_new
        if total > self.max_position:
            raise RequestRefused(f"request {rid!r}: context overflow, prompt {len(prompt)} + max_tokens {max_new} "
                                 f"exceeds {self.max_position} positions")
        need = self.manager.pages_needed_fresh(total)
        for g, (k, pool) in enumerate(zip(need, self.manager.pools)):
            window = self.manager.groups[g].window
            if window is not None:   # a windowed group holds at most the window, a portion and two partial pages
                P = self.manager.page_size
                k = min(k, -(-(window + self.config.largest_portion) // P) + 2)
            if k > pool.num_pages:
                raise RequestRefused(f"request {rid!r} can never fit: {k} pages needed in cache group {g}, the pool has {pool.num_pages}")
        seq = Sequence_(rid, prompt, max_new, arrival=self._arrivals, n_prompt_original=len(prompt),
                        priority=int(priority), arrival_time=self.clock())
        self._arrivals += 1
        self.waiting.append(seq)
        return seq

    def has_work(self) -> bool:
        return bool(self.waiting or self.running)

    def finish(self, seq: Sequence_) -> None:
        """The request is done (or aborted): its pages and slot return."""
        if seq in self.running:
            self.running.remove(seq)
            self.manager.free(seq.rid)
        else:
            try:
                self.waiting.remove(seq)
            except ValueError:
                pass

    # ---- one step -------------------------------------------------------------------
    def _preempt(self, victim: Sequence_) -> None:
        self.running.remove(victim)
        self.manager.free(victim.rid)
        victim.prompt = victim.prompt + victim.generated[victim.folded:]
        victim.folded = len(victim.generated)
        victim.computed = 0
        victim.admitted_at = -1
        victim.preemptions += 1
        self.waiting.appendleft(victim)

    def _reserve_or_preempt(self, seq: Sequence_, n: int, plan: StepPlan):
        """Pages for ``seq``'s next n tokens, preempting running requests if needed (the lowest priority first, the
        most recently admitted among equals).  Returns (whether ``seq`` got its pages: False when it had to go
        itself, the tokens of this step that victims already planned in it had been charged)."""
        refund = 0
        while True:
            try:
                self.manager.reserve(seq.rid, n)
                return True, refund
            except OutOfPages:
                victim = max(self.running, key=lambda s: (-s.priority, s.admitted_at))
                refund += sum(len(i.tokens) for i in plan.items if i.seq is victim)
                plan.items = [i for i in plan.items if i.seq is not victim]
                plan.preempted.append(victim.rid)
                self._preempt(victim)
                if victim is seq:
                    return False, refund

    def schedule(self) -> StepPlan:
        cfg = self.config
        plan = StepPlan([], [], [])
        budget = cfg.max_batch_tokens
        # portions are short for the sake of requests that decode beside them; with none, they may be long
        portion = cfg.chunked_prefill_tokens if any(not q.is_prefilling for q in self.running) else cfg.portion_alone
        # 1. running requests, oldest admission first (the list is kept in that order: admissions are appended,
        #    preemptions taken out): decodes cost one token, prompts a portion
        for seq in list(self.running):
            if budget <= 0 or (plan.preempted and seq not in self.running):   # nothing left to deal / preempted meanwhile
                continue
            if seq.is_prefilling:
                n = min(len(seq.prompt) - seq.computed, portion, budget)
                toks = seq.prompt[seq.computed: seq.computed + n]
                wants = seq.computed + n == len(seq.prompt)
            else:
                n, toks, wants = 1, [seq.generated[-1]], True
            ok, refund = self._reserve_or_preempt(seq, n, plan)
            budget += refund               # what a victim had been charged in this step is free again
            if ok:
                plan.items.append(PlannedItem(seq, toks, wants))
                budget -= n
        # 2. admissions, best score first (first come first served among equals); a request preempted in this step
        #    waits for the next
        now = self.clock()
        while self.waiting and len(self.running) < cfg.max_batch_size and budget > 0:
            seq = min(self.waiting, key=lambda q: (-self.score(q, now), q.arrival))
            if seq.rid in plan.preempted:
                break
            n = min(len(seq.prompt), portion, budget)
            need = self.manager.pages_needed_fresh(n)
            if any(k > f for k, f in zip(need, self.manager.free_pages())) or self.manager.free_slots() == 0:
                break
            self.waiting.remove(seq)
            self.manager.add(seq.rid)
            seq.admitted_at = self._admissions
            self._admissions += 1
            self.running.append(seq)
            plan.admitted.append(seq.rid)
            self.manager.reserve(seq.rid, n)
            plan.items.append(PlannedItem(seq, seq.prompt[:n], n == len(seq.prompt)))
            budget -= n
        return plan

    def advance(self, item: PlannedItem) -> None:
        """The step ran: the item's tokens are in the cache."""
        item.seq.computed += len(item.tokens)
