"""Accounting of the paged cache: pages, per-request block tables, layer groups, state slots.

This module owns no device memory and needs no GPU; it decides which page holds which token.
The tensors the pages index live in ``cache.storage``.  The bookkeeping itself is native code
(``csrc/cache_manager.cpp``, built on first use like the kernels); this file is its Python face:
it maps request ids to the slots the native side knows requests by, turns its error codes into
exceptions, and hands a step's arrays to numpy.

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

import ctypes
import dataclasses
from typing import Dict, Hashable, List, Optional, Sequence, Tuple

import numpy as np

from ..kernels.library import load_module

P = ctypes.c_void_p
I = ctypes.c_int


class OutOfPages(RuntimeError):
    """A group's pool cannot supply the pages a reservation needs.  Nothing was taken."""

    def __init__(self, group: int, needed: int, free: int):
        self.group, self.needed, self.free = group, needed, free
        super().__init__(f"cache group {group}: {needed} pages needed, {free} free")


class OutOfSlots(RuntimeError):
    """Every per-request state slot is taken."""


@dataclasses.dataclass(frozen=True)
class GroupSpec:
    """A set of schedule entries whose caches share pages.  ``window`` None keeps everything."""
    window: Optional[int]
    entries: Tuple[int, ...]


@dataclasses.dataclass
class RequestPages:
    """A copy of what the manager holds of one request."""
    length: int = 0                 # committed positions
    reserved: int = 0               # positions with pages, >= length
    tables: List[List[int]] = dataclasses.field(default_factory=list)  # per group
    state_slot: int = -1
    epoch: int = 0                  # differs between any two requests the manager ever had


class _Native:
    """The native library's functions with their C types, looked up once."""

    _fns = None

    @classmethod
    def get(cls):
        if cls._fns is None:
            mod = load_module("cache_manager")
            ip = ctypes.POINTER(ctypes.c_int)
            sig = {
                "cm_create": ((I, ip, ip, I, I), P), "cm_destroy": ((P,), None),
                "cm_pool_num_pages": ((P, I), I), "cm_pool_num_free": ((P, I), I), "cm_pool_take": ((P, I), I),
                "cm_pool_retain": ((P, I, I), I), "cm_pool_release": ((P, I, I), I), "cm_pool_refs": ((P, I, I), I),
                "cm_pool_free_list": ((P, I, ip), I), "cm_free_slots": ((P,), I), "cm_add": ((P,), I),
                "cm_free": ((P, I), I), "cm_length": ((P, I), I), "cm_reserved": ((P, I), I),
                "cm_epoch": ((P, I), ctypes.c_longlong), "cm_pages_needed": ((P, I, I, ip), I),
                "cm_can_reserve": ((P, ip, ip, I, ip), I), "cm_reserve": ((P, I, I, ip), I), "cm_commit": ((P, I, I), I),
                "cm_table_len": ((P, I, I), I), "cm_table": ((P, I, I, ip, I), I),
                "cm_commit_each": ((P, ip, I, I), I), "cm_unchanged": ((P, ip, ctypes.POINTER(ctypes.c_longlong), ip, I), I),
                "cm_step_widths": ((P, ip, I, I, ip), I),
                "cm_step_fill": ((P, ip, ip, I, ip, ip, ip, ip, ip, ip, ip, ip), I), "cm_check": ((P,), I),
            }
            fns = {}
            for name, (args, res) in sig.items():
                f = getattr(mod.lib, name)
                f.argtypes, f.restype = list(args), res
                fns[name] = f
            fns["last_error"] = mod.last_error
            cls._fns = type("NativeCacheManager", (), fns)
        return cls._fns


def _ints(values) -> "ctypes.Array":
    return (ctypes.c_int * len(values))(*values)


def _ptr(a: np.ndarray):
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_int))


class PagePool:
    """Pages 0..n-1 with reference counts; free pages are reused most-recently-freed first.  Alone it owns a
    native manager of one group; the manager's own pools are views of its groups."""

    def __init__(self, num_pages: int, _owner=None, _group: int = 0):
        self._n = _Native.get()
        if _owner is None:
            if num_pages <= 0:
                raise ValueError("a pool needs at least one page")
            self._h = self._n.cm_create(1, _ints([num_pages]), _ints([-1]), 1, 0)
            self._owned = True
        else:
            self._h, self._owned = _owner, False
        self._g = _group
        self.num_pages = self._n.cm_pool_num_pages(self._h, self._g)

    def __del__(self):
        if getattr(self, "_owned", False) and self._h:
            self._n.cm_destroy(self._h)
            self._h = None

    @property
    def num_free(self) -> int:
        return self._n.cm_pool_num_free(self._h, self._g)

    @property
    def _free(self) -> List[int]:
        out = np.empty(max(self.num_pages, 1), dtype=np.int32)
        n = self._n.cm_pool_free_list(self._h, self._g, _ptr(out))
        return out[:n].tolist()

    def take(self) -> int:
        p = self._n.cm_pool_take(self._h, self._g)
        if p < 0:
            raise OutOfPages(-1, 1, 0)
        return p

    def retain(self, page: int) -> None:
        if self._n.cm_pool_retain(self._h, self._g, int(page)) != 0:
            raise ValueError(self._n.last_error())

    def release(self, page: int) -> None:
        if self._n.cm_pool_release(self._h, self._g, int(page)) != 0:
            raise ValueError(self._n.last_error())

    def refs(self, page: int) -> int:
        return self._n.cm_pool_refs(self._h, self._g, int(page))


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
        if any(n <= 0 for n in counts):
            raise ValueError("a pool needs at least one page")
        self._n = _Native.get()
        windows = [-1 if g.window is None else int(g.window) for g in self.groups]
        self._h = self._n.cm_create(len(counts), _ints(counts), _ints(windows), page_size, max_requests)
        if not self._h:
            raise ValueError(self._n.last_error())
        self.pools = [PagePool(n, _owner=self._h, _group=g) for g, n in enumerate(counts)]
        self.max_requests = max_requests
        self._slot: Dict[Hashable, int] = {}        # live request -> its slot, which is how the native side knows it
        self._need = (ctypes.c_int * max(len(counts), 1))()
        self._fail = (ctypes.c_int * 3)()
        # Called with the slot of every request that is added, whoever adds it (the runner for a replayed
        # trace, the scheduler for an admission or a re-admission after preemption): the storage hangs the
        # clearing of per-request state here, so that no path can hand out a slot with its last owner's state.
        self.on_add = None

    def __del__(self):
        if getattr(self, "_h", None):
            self._n.cm_destroy(self._h)
            self._h = None

    # ---- requests -------------------------------------------------------------------
    def has(self, rid: Hashable) -> bool:
        return rid in self._slot

    def live(self) -> List[Hashable]:
        return list(self._slot)

    def add(self, rid: Hashable) -> int:
        if rid in self._slot:
            raise ValueError(f"request {rid!r} is already live")
        slot = self._n.cm_add(self._h)
        if slot < 0:
            raise OutOfSlots(f"all {self.max_requests} request slots are in use")
        self._slot[rid] = slot
        if self.on_add is not None:
            self.on_add(slot)
        return slot

    def _slot_of(self, rid: Hashable) -> int:
        try:
            return self._slot[rid]
        except KeyError:
            raise KeyError(f"request {rid!r} is not live") from None

    def get(self, rid: Hashable) -> RequestPages:
        s = self._slot_of(rid)
        return RequestPages(self._n.cm_length(self._h, s), self._n.cm_reserved(self._h, s),
                            [self.block_table(rid, g) for g in range(len(self.groups))], s, self._n.cm_epoch(self._h, s))

    def epoch(self, rid: Hashable) -> int:
        """A number that tells this live request from every other the manager ever had, or -1 if it is not live."""
        s = self._slot.get(rid)
        return -1 if s is None else self._n.cm_epoch(self._h, s)

    def length(self, rid: Hashable) -> int:
        return self._n.cm_length(self._h, self._slot_of(rid))

    def free(self, rid: Hashable) -> None:
        s = self._slot.pop(rid, None)
        if s is None:
            raise KeyError(f"request {rid!r} is not live (freed twice?)")
        if self._n.cm_free(self._h, s) != 0:
            raise RuntimeError(self._n.last_error())

    # ---- pages ----------------------------------------------------------------------
    def _blocks_for(self, positions: int) -> int:
        return (positions + self.page_size - 1) // self.page_size

    def pages_needed(self, rid: Hashable, n_new: int) -> List[int]:
        """New pages per group to hold the request's next ``n_new`` positions."""
        self._n.cm_pages_needed(self._h, self._slot_of(rid), int(n_new), self._need)
        return list(self._need[:len(self.groups)])

    def pages_needed_fresh(self, n_tokens: int) -> List[int]:
        """Pages per group a request that holds nothing needs for its first ``n_tokens``."""
        return [self._blocks_for(n_tokens)] * len(self.groups)

    def free_pages(self) -> List[int]:
        return [p.num_free for p in self.pools]

    def free_slots(self) -> int:
        return self._n.cm_free_slots(self._h)

    def can_reserve(self, needs: Sequence[Tuple[Hashable, int]], totals: Optional[List[int]] = None) -> bool:
        """Whether all of ``needs`` [(request, n_new)] fit at once.  ``totals`` (a list) receives the pages
        they need per group."""
        slots = _ints([self._slot_of(rid) for rid, _ in needs])
        ns = _ints([int(n) for _, n in needs])
        ok = self._n.cm_can_reserve(self._h, slots, ns, len(needs), self._need)
        if totals is not None:
            totals[:] = list(self._need[:len(self.groups)])
        return ok == 1

    def reserve(self, rid: Hashable, n_new: int) -> None:
        """Give the request pages for positions [length, length + n_new) in every group, or
        raise OutOfPages and change nothing."""
        if n_new <= 0:
            raise ValueError("reserve needs a positive token count")
        rc = self._n.cm_reserve(self._h, self._slot_of(rid), int(n_new), self._fail)
        if rc == 1:
            raise OutOfPages(*self._fail[:3])
        if rc != 0:
            raise RuntimeError(self._n.last_error())

    def commit(self, rid: Hashable, n_new: int) -> None:
        """The step that wrote ``n_new`` positions has run: they count now.  Windowed groups give
        back every page whose positions all lie before the window of the next query."""
        if self._n.cm_commit(self._h, self._slot_of(rid), int(n_new)) != 0:
            raise ValueError(f"request {rid!r}: {self._n.last_error()}")

    def commit_each(self, rids: Sequence[Hashable], n_new: int) -> None:
        """``commit(rid, n_new)`` for every request of the list, in one call."""
        slots = _ints([self._slot_of(r) for r in rids])
        if self._n.cm_commit_each(self._h, slots, len(rids), int(n_new)) != 0:
            raise ValueError(self._n.last_error())

    def snapshot(self, rids: Sequence[Hashable]):
        """What ``unchanged`` compares later: the requests' slots, epochs and lengths."""
        slots = [self._slot_of(r) for r in rids]
        return (list(rids), _ints(slots), (ctypes.c_longlong * len(slots))(*[self._n.cm_epoch(self._h, s) for s in slots]),
                _ints([self._n.cm_length(self._h, s) for s in slots]))

    @staticmethod
    def snapshot_rows(snapshot, rows: Sequence[int]):
        """The snapshot of only the requests at places ``rows`` of ``snapshot``."""
        was, slots, epochs, lengths = snapshot
        return ([was[i] for i in rows], _ints([slots[i] for i in rows]),
                (ctypes.c_longlong * len(rows))(*[epochs[i] for i in rows]), _ints([lengths[i] for i in rows]))

    def unchanged(self, snapshot, rids: Sequence[Hashable]) -> bool:
        """Whether ``rids`` are the requests of the snapshot, in its order, all still live and none of them moved."""
        was, slots, epochs, lengths = snapshot
        if len(was) != len(rids) or any(a != b for a, b in zip(was, rids)):
            return False
        return self._n.cm_unchanged(self._h, slots, epochs, lengths, len(was)) == 1

    def block_table(self, rid: Hashable, group: int) -> List[int]:
        s = self._slot_of(rid)
        n = self._n.cm_table_len(self._h, s, group)
        out = np.empty(max(n, 1), dtype=np.int32)
        self._n.cm_table(self._h, s, group, _ptr(out), n)
        return out[:n].tolist()

    def slot_of(self, rid: Hashable, group: int, position: int) -> int:
        """page * page_size + offset of ``position`` (must hold a page)."""
        page = self.block_table(rid, group)[position // self.page_size]
        if page < 0:
            raise ValueError(f"request {rid!r}: position {position} of group {group} has been released")
        return page * self.page_size + position % self.page_size

    def state_slot(self, rid: Hashable) -> int:
        return self._slot_of(rid)

    # ---- a step's arrays ------------------------------------------------------------
    def step_arrays(self, rids: Sequence[Hashable], q_len: Sequence[int], width_multiple: int):
        """For a step in which request ``rids[i]`` brings ``q_len[i]`` tokens, rows laid end to end: a dict of int32
        arrays ``start`` (the requests' lengths), ``q_start``, ``kv_len``, ``state_slots`` [R]; ``row_req``,
        ``positions`` [T]; and per group ``block_tables`` [R, width] (-1 where no page; width a multiple of
        ``width_multiple``) and ``write_slots`` [T] (page * page_size + offset of every row's key and value)."""
        R, G = len(rids), len(self.groups)
        slots = np.array([self._slot_of(r) for r in rids], dtype=np.int32)
        q = np.asarray(q_len, dtype=np.int32)
        T = int(q.sum())
        widths = np.empty(max(G, 1), dtype=np.int32)
        if self._n.cm_step_widths(self._h, _ptr(slots), R, int(width_multiple), _ptr(widths)) != 0:
            raise KeyError(self._n.last_error())
        start, q_start, kv_len = (np.empty(max(R, 1), dtype=np.int32)[:R] for _ in range(3))
        row_req, positions = (np.empty(max(T, 1), dtype=np.int32)[:T] for _ in range(2))
        tables = np.empty(max(int(R * widths[:G].sum()), 1), dtype=np.int32)
        write_slots = np.empty(max(G * T, 1), dtype=np.int32)
        rc = self._n.cm_step_fill(self._h, _ptr(slots), _ptr(q), R, _ptr(widths), _ptr(start), _ptr(q_start), _ptr(kv_len),
                                  _ptr(row_req), _ptr(positions), _ptr(tables), _ptr(write_slots))
        if rc <= -2:
            raise RuntimeError(f"cache group {-rc - 2}: a row of this step has no page (reserve before building the step)")
        if rc < 0:
            raise KeyError(self._n.last_error())
        bts, off = [], 0
        for g in range(G):
            w = int(widths[g])
            bts.append(tables[off:off + R * w].reshape(R, w))
            off += R * w
        return {"start": start, "q_start": q_start, "q_len": q, "kv_len": kv_len, "state_slots": slots, "row_req": row_req,
                "positions": positions, "block_tables": bts,
                "write_slots": [write_slots[g * T:(g + 1) * T] for g in range(G)]}

    # ---- invariants (tests call this after every operation) ---------------------------
    def check(self) -> None:
        assert self._n.cm_check(self._h) == 0, self._n.last_error()
        assert len(set(self._slot.values())) == len(self._slot), "two requests share a slot"
        assert len(self._slot) + self.free_slots() == self.max_requests, "state slots lost"
