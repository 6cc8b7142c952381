"""What one step looks like to the parts: the flattened rows of a batch and their metadata.

A step is a list of (request, its next tokens).  All rows are laid end to end; the rows of one
request are contiguous and in position order.  For every row the context gives its token,
its absolute position and its request's index in the batch; for every request its row range,
its length after the step and its state slot; for every cache group the block tables and the
slot each row's key and value are written to.  Everything is built on the host as int32 and
uploaded in one copy.

The reference passes a list of UnifiedBatchInput{sequence_id, n_past, tokens, request_logits}
(runtime/backends/common/backend_types.h:22-34) and splits it into one batched decode forward
plus one forward per prefill item (runtime/backends/cuda/inferflux_cuda_executor.cpp:3231-3263,
3289-3345, 3539-3625); here the whole list is one forward.
"""
from __future__ import annotations

import dataclasses
from typing import Callable, Dict, Hashable, List, Sequence

import numpy as np
import torch


@dataclasses.dataclass
class StepEntry:
    """A request's share of a step: its next ``tokens`` and the places among them (indices into
    ``tokens``) whose logits are wanted."""
    rid: Hashable
    tokens: Sequence[int]
    want: Sequence[int] = ()


def _pad_arrays(arrays, n_pad: int, scratch_pages: Sequence[int], page_size: int, scratch_state_slot: int = 0):
    """``arrays`` of a step (``CacheManager.step_arrays``) with ``n_pad`` rows that stand for nobody appended: each is
    a request of its own with one token at position 0 whose key and value go to the group's scratch page (a page
    outside every pool, which nobody's block table names) and which reads that one key back; a mixer with state of
    its own is given ``scratch_state_slot`` for them (a slot no request ever holds).  Such rows keep a step's layout
    the same while the number of real requests changes; what they compute is thrown away."""
    R, T = arrays["q_len"].shape[0], arrays["positions"].shape[0]
    i32 = lambda v: np.asarray(v, dtype=np.int32)
    out = dict(arrays)
    out["start"] = np.concatenate([arrays["start"], np.zeros(n_pad, np.int32)])
    out["q_start"] = np.concatenate([arrays["q_start"], i32(np.arange(T, T + n_pad))])
    out["q_len"] = np.concatenate([arrays["q_len"], np.ones(n_pad, np.int32)])
    out["kv_len"] = np.concatenate([arrays["kv_len"], np.ones(n_pad, np.int32)])
    out["state_slots"] = np.concatenate([arrays["state_slots"], np.full(n_pad, scratch_state_slot, np.int32)])
    out["row_req"] = np.concatenate([arrays["row_req"], i32(np.arange(R, R + n_pad))])
    out["positions"] = np.concatenate([arrays["positions"], np.zeros(n_pad, np.int32)])
    tables, slots = [], []
    for g, bt in enumerate(arrays["block_tables"]):
        pad = np.full((n_pad, bt.shape[1]), -1, np.int32)
        pad[:, 0] = scratch_pages[g]
        tables.append(np.concatenate([bt, pad]))
        slots.append(np.concatenate([arrays["write_slots"][g], i32(scratch_pages[g] * page_size + np.arange(n_pad) % page_size)]))
    out["block_tables"], out["write_slots"] = tables, slots
    return out


class StepContext:
    """``width_multiple`` rounds the block tables' width up (a replayed graph needs the same layout
    for many steps).  ``slab`` is a device buffer to fill instead of a new one, ``pinned`` the host
    buffer the copy goes through; ``layout_key`` tells whether two steps have the same layout.
    ``pad_requests`` appends that many rows that stand for nobody (see ``_pad_arrays``; ``scratch_pages``: per
    cache group the page they write to, ``scratch_state_slot``: the state slot they use); their logits come last and
    are the caller's to drop.  ``n_requests``
    and ``n_tokens`` count them, ``n_real_requests`` and ``n_real_tokens`` do not."""

    def __init__(self, entries: Sequence[StepEntry], manager, act_dtype: torch.dtype, device,
                 width_multiple: int = 8, slab: torch.Tensor = None, pinned: torch.Tensor = None, upload: bool = True,
                 pad_requests: int = 0, scratch_pages: Sequence[int] = (), scratch_state_slot: int = 0):
        self.act_dtype, self.device = act_dtype, device
        self.timer = None              # a tracing.PhaseTimer while per-phase timing is on
        self.entries = list(entries)
        self.n_real_requests = len(self.entries)
        # lengths, positions, block tables and write slots come from the cache manager's native side in one call
        arrays = manager.step_arrays([e.rid for e in self.entries], [len(e.tokens) for e in self.entries], width_multiple)
        self.n_real_tokens = int(arrays["positions"].shape[0])
        if pad_requests > 0:
            if len(scratch_pages) != len(manager.groups):
                raise ValueError("padding rows need a scratch page for every cache group")
            arrays = _pad_arrays(arrays, pad_requests, scratch_pages, manager.page_size, scratch_state_slot)
        R = self.n_requests = self.n_real_requests + max(pad_requests, 0)
        q_len, q_start, start = arrays["q_len"], arrays["q_start"], arrays["start"]
        T = self.n_tokens = int(arrays["positions"].shape[0])
        self.h_q_len, self.h_q_start, self.h_start_pos = q_len, q_start, start
        self.h_kv_len = arrays["kv_len"]
        self.h_token_ids = np.concatenate([np.asarray(e.tokens, dtype=np.int32) for e in self.entries]
                                          + [np.zeros(max(pad_requests, 0), np.int32)]) if R else np.zeros(0, np.int32)
        self.h_row_req, self.h_positions = arrays["row_req"], arrays["positions"]
        rows: List[int] = []
        for i, e in enumerate(self.entries):
            rows.extend(int(q_start[i]) + int(w) for w in e.want)
        self.n_real_logit_rows = len(rows)
        rows.extend(range(self.n_real_tokens, T))            # rows that stand for nobody: last, dropped by the caller
        self.h_logit_rows = np.asarray(rows, dtype=np.int32)
        self.n_logit_rows = len(rows)
        # every row of the step wants its logits, in order (a step of single tokens): the rows that the last product of the
        # layers prepares for the final norm are then the head's input as they are
        self.all_rows_wanted = rows == list(range(T))
        self.h_state_slots = arrays["state_slots"]
        n_groups = len(manager.groups)
        self.h_block_tables: List[np.ndarray] = arrays["block_tables"]
        self.h_write_slots: List[np.ndarray] = arrays["write_slots"]

        # One upload: every array above, end to end, each start aligned to 4 ints.
        named = [("token_ids", self.h_token_ids), ("positions", self.h_positions), ("row_req", self.h_row_req),
                 ("q_start", q_start), ("q_len", q_len), ("kv_len", self.h_kv_len),
                 ("logit_rows", self.h_logit_rows), ("state_slots", self.h_state_slots)]
        for g in range(n_groups):
            named.append((f"block_table{g}", self.h_block_tables[g]))
            named.append((f"write_slots{g}", self.h_write_slots[g]))
        offs, total = {}, 0
        for name, a in named:
            offs[name] = (total, a.size, a.shape)
            total += (a.size + 3) // 4 * 4
        self.layout_key = (R, T, self.n_logit_rows, tuple(bt.shape[1] for bt in self.h_block_tables))
        # No request of this step holds more positions than its block table has room for.  Kernels size
        # their grids by this bound, not by the lengths themselves, so that a captured step stays valid
        # while lengths grow within the same table width.
        self.kv_bound = max((bt.shape[1] for bt in self.h_block_tables), default=0) * manager.page_size
        self.slab_size = max(total, 4)
        self._named, self._offs = named, offs
        self._views: Dict[str, torch.Tensor] = {}
        self._derived: Dict[object, object] = {}
        self._slab = None
        if upload:
            self.bind(slab, pinned)

    def set_tokens(self, entries: Sequence[StepEntry], tokens: Sequence[int]) -> None:
        """For a context built ahead of its tokens (one placeholder token per request): the step's entries and
        their tokens, before ``bind``."""
        if len(tokens) != self.n_real_tokens or len(entries) != self.n_real_requests:
            raise ValueError("set_tokens: not the step this context was built for")
        self.entries = list(entries)
        self.h_token_ids[:self.n_real_tokens] = tokens

    def bind(self, slab: torch.Tensor = None, pinned: torch.Tensor = None) -> None:
        """Put the step's arrays on the device: into ``slab`` through ``pinned`` when given (an
        asynchronous copy on the current stream), else into a new tensor."""
        if pinned is not None:
            host = pinned.numpy()
        else:
            host = np.zeros(self.slab_size, dtype=np.int32)
        self.write_host(host)
        if slab is None:
            slab = torch.from_numpy(host).to(self.device)
        elif pinned is not None:
            slab.copy_(pinned, non_blocking=True)
        else:
            slab.copy_(torch.from_numpy(host))
        self.use_slab(slab)

    def write_host(self, host: np.ndarray) -> None:
        """The step's arrays, end to end, into ``host`` (int32, at least ``slab_size`` long)."""
        for name, a in self._named:
            o, n, _ = self._offs[name]
            host[o:o + n] = a.reshape(-1)

    def use_slab(self, slab: torch.Tensor) -> None:
        """Take ``slab`` (which already holds a step of this layout) as the device arrays."""
        self._slab = slab
        self._views = {}
        for name, _ in self._named:
            o, n, shape = self._offs[name]
            self._views[name] = slab[o:o + n].view(shape)
        self._derived = {}

    # ---- device views -------------------------------------------------------------
    @property
    def token_ids(self) -> torch.Tensor: return self._views["token_ids"]
    @property
    def positions(self) -> torch.Tensor: return self._views["positions"]
    @property
    def row_req(self) -> torch.Tensor: return self._views["row_req"]
    @property
    def q_start(self) -> torch.Tensor: return self._views["q_start"]
    @property
    def q_len(self) -> torch.Tensor: return self._views["q_len"]
    @property
    def kv_len(self) -> torch.Tensor: return self._views["kv_len"]
    @property
    def logit_rows(self) -> torch.Tensor: return self._views["logit_rows"]
    @property
    def state_slots(self) -> torch.Tensor: return self._views["state_slots"]

    def block_table(self, group: int) -> torch.Tensor:
        return self._views[f"block_table{group}"]

    def write_slots(self, group: int) -> torch.Tensor:
        return self._views[f"write_slots{group}"]

    def derived(self, key, make: Callable[[], object]):
        """A value computed once per step and shared by every layer that asks (kernel work lists)."""
        if key not in self._derived:
            self._derived[key] = make()
        return self._derived[key]

    def upload(self, array: np.ndarray) -> torch.Tensor:
        return torch.from_numpy(np.ascontiguousarray(array)).to(self.device)
