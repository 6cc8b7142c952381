"""The cache manager's accounting in plain Python: what the native manager (inferflux_amd/csrc/cache_manager.cpp)
is compared with, operation by operation, in test_cache_manager.py.  It shares no code with it.

It decides which page holds which token: pages, per-request block tables, layer groups, state slots.

Layers whose mixers keep the same kind of history form a *group*: all layers that keep every
key share one group, all layers that keep a window of W keys share another.  Each group has
its own pool of pages and, for every request, its own block table: entry b is the page that
holds positions [b * page_size, (b + 1) * page_size) for every layer of the group, or -1 once
a windowed group has given that page back.

A request's life: ``add`` (takes a state slot), then per step ``reserve(n)`` (pages for its
next n positions in every group, all or nothing) and, after the step ran, ``commit(n)``
(the positions now count; a windowed group releases pages no later query can see), finally
``free`` (everything returns).  A page goes back to its pool's free list the moment its
reference count reaches zero and is handed out again, most recently freed first.

The reference accounts pages on the host in the same units (16-token blocks, reference counts:
runtime/kv_cache/paged_kv_cache.cpp:40-86, 360-371; scheduler/scheduler.cpp:293, 2327-2335)
but its GPU cache is one contiguous slot per sequence that the kernels address without the
table (runtime/backends/cuda/native/kv_cache_gpu.cu:21-78).  It has no groups and no state
slots; its nearest thing to per-request state is the penalty history kept per slot
(runtime/backends/cuda/inferflux_cuda_executor.h:353-357).
"""
from __future__ import annotations

import dataclasses
from typing import Dict, Hashable, List, Optional, Sequence, Tuple


class OutOfPages(RuntimeError):
    """A group's pool cannot supply the pages a reservation needs.  Nothing was taken."""

    def __init__(self, group: int, needed: int, free: int):
        self.group, self.needed, self.free = group, needed, free
        super().__init__(f"cache group {group}: {needed} pages needed, {free} free")


class OutOfSlots(RuntimeError):
    """Every per-request state slot is taken."""


class PagePool:
    """Pages 0..n-1 with reference counts; free pages are reused most-recently-freed first."""

    def __init__(self, num_pages: int):
        if num_pages <= 0:
            raise ValueError("a pool needs at least one page")
        self.num_pages = num_pages
        self._free: List[int] = list(range(num_pages - 1, -1, -1))  # pop() hands out page 0 first
        self._refs: List[int] = [0] * num_pages

    @property
    def num_free(self) -> int:
        return len(self._free)

    def take(self) -> int:
        if not self._free:
            raise OutOfPages(-1, 1, 0)
        p = self._free.pop()
        assert self._refs[p] == 0, f"page {p} on the free list is still referenced"
        self._refs[p] = 1
        return p

    def retain(self, page: int) -> None:
        if self._refs[page] <= 0:
            raise ValueError(f"page {page} is not in use")
        self._refs[page] += 1

    def release(self, page: int) -> None:
        if not (0 <= page < self.num_pages) or self._refs[page] <= 0:
            raise ValueError(f"page {page} released but not in use (freed twice?)")
        self._refs[page] -= 1
        if self._refs[page] == 0:
            self._free.append(page)

    def refs(self, page: int) -> int:
        return self._refs[page]


@dataclasses.dataclass(frozen=True)
class GroupSpec:
    """A set of schedule entries whose caches share pages.  ``window`` None keeps everything."""
    window: Optional[int]
    entries: Tuple[int, ...]


@dataclasses.dataclass
class RequestPages:
    length: int = 0                 # committed positions
    reserved: int = 0               # positions with pages, >= length
    tables: List[List[int]] = dataclasses.field(default_factory=list)  # per group
    state_slot: int = -1


class CacheManager:
    def __init__(self, groups: Sequence[GroupSpec], page_size: int, num_pages, max_requests: int):
        """``num_pages``: one number for every group, or one per group."""
        if page_size <= 0:
            raise ValueError("page_size must be positive")
        self.groups = list(groups)
        self.page_size = page_size
        counts = [num_pages] * len(self.groups) if isinstance(num_pages, int) else list(num_pages)
        if len(counts) != len(self.groups):
            raise ValueError("one page count per group expected")
        self.pools = [PagePool(n) for n in counts]
        self.max_requests = max_requests
        self._free_slots: List[int] = list(range(max_requests - 1, -1, -1))
        self._requests: Dict[Hashable, RequestPages] = {}

    # ---- requests -------------------------------------------------------------------
    def has(self, rid: Hashable) -> bool:
        return rid in self._requests

    def live(self) -> List[Hashable]:
        return list(self._requests)

    def add(self, rid: Hashable) -> int:
        """Start a request; returns its state slot (the caller zeroes the slot's state)."""
        if rid in self._requests:
            raise ValueError(f"request {rid!r} is already live")
        if not self._free_slots:
            raise OutOfSlots(f"all {self.max_requests} request slots are in use")
        r = RequestPages(tables=[[] for _ in self.groups], state_slot=self._free_slots.pop())
        self._requests[rid] = r
        return r.state_slot

    def get(self, rid: Hashable) -> RequestPages:
        try:
            return self._requests[rid]
        except KeyError:
            raise KeyError(f"request {rid!r} is not live") from None

    def peek(self, rid: Hashable) -> Optional[RequestPages]:
        """The live request's record, or None."""
        return self._requests.get(rid)

    def length(self, rid: Hashable) -> int:
        return self.get(rid).length

    def free(self, rid: Hashable) -> None:
        r = self._requests.pop(rid, None)
        if r is None:
            raise KeyError(f"request {rid!r} is not live (freed twice?)")
        for g, table in enumerate(r.tables):
            for p in table:
                if p >= 0:
                    self.pools[g].release(p)
        self._free_slots.append(r.state_slot)

    # ---- pages ----------------------------------------------------------------------
    def _blocks_for(self, positions: int) -> int:
        return (positions + self.page_size - 1) // self.page_size

    def pages_needed(self, rid: Hashable, n_new: int) -> List[int]:
        """New pages per group to hold the request's next ``n_new`` positions."""
        r = self.get(rid)
        return [max(0, self._blocks_for(r.length + n_new) - len(t)) for t in r.tables]

    def pages_needed_fresh(self, n_tokens: int) -> List[int]:
        """Pages per group a request that holds nothing needs for its first ``n_tokens``."""
        return [self._blocks_for(n_tokens)] * len(self.groups)

    def free_pages(self) -> List[int]:
        return [p.num_free for p in self.pools]

    def free_slots(self) -> int:
        return len(self._free_slots)

    def can_reserve(self, needs: Sequence[Tuple[Hashable, int]]) -> bool:
        """Whether all of ``needs`` [(request, n_new)] fit at once."""
        tot = [0] * len(self.groups)
        for rid, n in needs:
            for g, k in enumerate(self.pages_needed(rid, n)):
                tot[g] += k
        return all(t <= p.num_free for t, p in zip(tot, self.pools))

    def reserve(self, rid: Hashable, n_new: int) -> None:
        """Give the request pages for positions [length, length + n_new) in every group, or
        raise OutOfPages and change nothing."""
        if n_new <= 0:
            raise ValueError("reserve needs a positive token count")
        r = self.get(rid)
        need = self.pages_needed(rid, n_new)
        for g, k in enumerate(need):
            if k > self.pools[g].num_free:
                raise OutOfPages(g, k, self.pools[g].num_free)
        for g, k in enumerate(need):
            for _ in range(k):
                r.tables[g].append(self.pools[g].take())
        r.reserved = max(r.reserved, r.length + n_new)

    def commit(self, rid: Hashable, n_new: int) -> None:
        """The step that wrote ``n_new`` positions has run: they count now.  Windowed groups give
        back every page whose positions all lie before the window of the next query."""
        r = self.get(rid)
        if r.length + n_new > r.reserved:
            raise ValueError(f"request {rid!r}: commit of {n_new} beyond the {r.reserved - r.length} reserved positions")
        r.length += n_new
        for g, spec in enumerate(self.groups):
            if spec.window is None:
                continue
            first_needed = r.length - spec.window + 1  # oldest position the next query reads
            if first_needed <= 0:
                continue
            dead_blocks = min(first_needed // self.page_size, len(r.tables[g]))
            t = r.tables[g]
            for b in range(dead_blocks - 1, -1, -1):  # released blocks form a prefix: stop at the first -1
                if t[b] < 0:
                    break
                self.pools[g].release(t[b])
                t[b] = -1

    def block_table(self, rid: Hashable, group: int) -> List[int]:
        return self.get(rid).tables[group]

    def slot_of(self, rid: Hashable, group: int, position: int) -> int:
        """page * page_size + offset of ``position`` (must hold a page)."""
        page = self.get(rid).tables[group][position // self.page_size]
        if page < 0:
            raise ValueError(f"request {rid!r}: position {position} of group {group} has been released")
        return page * self.page_size + position % self.page_size

    def state_slot(self, rid: Hashable) -> int:
        return self.get(rid).state_slot

    # ---- invariants (tests call this after every operation) ---------------------------
    def check(self) -> None:
        for g, pool in enumerate(self.pools):
            held: Dict[int, int] = {}
            for rid, r in self._requests.items():
                for p in r.tables[g]:
                    if p >= 0:
                        held[p] = held.get(p, 0) + 1
            free = pool._free
            assert len(set(free)) == len(free), f"group {g}: a page is on the free list twice"
            assert not (set(free) & set(held)), f"group {g}: a page is both free and held"
            assert len(free) + len(held) == pool.num_pages, f"group {g}: pages lost ({len(free)} free + {len(held)} held != {pool.num_pages})"
            for p, n in held.items():
                assert pool.refs(p) == n, f"group {g}: page {p} held {n} times with {pool.refs(p)} references"
        slots = [r.state_slot for r in self._requests.values()]
        assert len(set(slots)) == len(slots), "a state slot is held twice"
        assert not (set(slots) & set(self._free_slots)), "a state slot is both free and held"
        assert len(slots) + len(self._free_slots) == self.max_requests, "state slots lost"
