"""The step function: run a batch of (request, next tokens) from the cache and return logits.

``ModelRunner.step`` takes any mix of prompt portions and single decoded tokens, cut anywhere.
It checks the whole step first (known requests, token ids, positions, pages), reserves pages
for every row or raises before anything has changed, runs all rows as one batch, commits the
new positions and returns float32 logits at the wanted places, in the order of the entries
and of their ``want`` lists.  It samples nothing.

The reference's step (InferfluxCudaExecutor::ExecuteUnifiedBatch,
runtime/backends/cuda/inferflux_cuda_executor.cpp:3165-3769) samples inside the step and
reports failures per item (3234-3253, 3545-3560); here a step succeeds for every entry or
raises before it touches the cache.
"""
from __future__ import annotations

import os
from typing import Hashable, Optional, Sequence

import torch

from ..cache.manager import OutOfPages
from ..cache.storage import CacheStorage
from ..kernels import ops
from .context import StepContext, StepEntry
from .model import Model


class StepError(ValueError):
    """A step that cannot run; the cache is unchanged."""


class _DecodeGraph:
    """A captured decode step: the device arrays it reads, the host buffer they are filled through,
    the graph and the logits it writes."""

    def __init__(self, slab, pinned, graph, ctx, logits):
        self.slab, self.pinned, self.graph, self.ctx, self.logits = slab, pinned, graph, ctx, logits
        self.host = pinned.numpy()      # the pinned buffer as the array the step's arrays are written into
        self.copied = torch.cuda.Event()


class ModelRunner:
    GRAPH_WIDTH_MULTIPLE = 64     # block-table width (pages) a captured step is valid for, in steps of this
    MAX_GRAPHS = 24               # captured layouts kept; the one unused longest goes first
    # A captured step is valid for one number of rows.  A batch that shrinks a request at a time would need a capture
    # (a wait for the GPU, an eager step, the capture: tens of milliseconds) for every size it passes through, so the
    # batch of a captured step is filled up to the next of these sizes with rows that stand for nobody (they write
    # to a scratch page and their logits are dropped).  The sizes follow the products' kernels (up to 16 rows one
    # kernel, 17-64 another) and cost nothing there: a weight-streaming product reads the same bytes for 5 rows and 8.
    GRAPH_BATCH_SIZES = (1, 2, 4, 8, 16, 24, 32, 48, 64)

    def __init__(self, model: Model, num_pages: int, page_size: int = 16, max_requests: int = 64,
                 decode_graphs: bool = True, phase_timing: bool = False):
        if model.device is None:
            raise ValueError("the model has no weights yet (load_folder / init_random first)")
        if model.device.type != "cuda":
            raise RuntimeError(f"the engine runs on the GPU only, the model is on {model.device}")
        self.model = model
        self.device, self.dtype = model.device, model.dtype
        self.storage = CacheStorage(model.plan.schedule, model.schedule_mixers(), page_size, num_pages,
                                    max_requests, model.dtype, model.device)
        self.manager = self.storage.manager
        self.page_size = page_size
        self.vocab_size = model.plan.vocab_size
        self.max_position = model.plan.max_position
        # Steps in which every request brings one token are captured as HIP graphs, one per layout
        # (batch size, wanted rows, block-table width), and replayed: a decode step is some 250
        # launches, which the host cannot issue as fast as the GPU runs them.  The reference does the
        # same per batch size (runtime/backends/cuda/native/transformer_forward.cu:3068-3117).
        self.timer = None
        if phase_timing or os.environ.get("INFERFLUX_PHASE_TIMING", "") == "1":
            from .tracing import PhaseTimer
            self.timer = PhaseTimer()
        self.decode_graphs = decode_graphs and model.graph_safe and self.timer is None
        self._graphs = {}
        self.graph_captures = 0    # decode-step layouts captured so far (each costs an eager step, a wait for the GPU and a capture)
        self.graph_replays = 0
        self._prepared = None      # (the manager's snapshot of the requests, the context) of a step got ready ahead of its tokens
        self._launched = None      # (that snapshot, the graph) of a step already started with tokens the host has not seen

    # ---- requests -----------------------------------------------------------------
    def add_request(self, rid: Hashable) -> None:
        self.manager.add(rid)          # (the storage clears the slot's per-request state as the manager hands it out)

    def free_request(self, rid: Hashable) -> None:
        self.manager.free(rid)

    def has_request(self, rid: Hashable) -> bool:
        return self.manager.has(rid)

    def length(self, rid: Hashable) -> int:
        return self.manager.length(rid)

    # ---- the step -----------------------------------------------------------------
    def validate(self, entries: Sequence[StepEntry]) -> None:
        seen = set()
        for e in entries:
            if e.rid in seen:
                raise StepError(f"request {e.rid!r} appears twice in one step")
            seen.add(e.rid)
            if not self.manager.has(e.rid):
                raise StepError(f"request {e.rid!r} is not live (add_request first)")
            n = len(e.tokens)
            if n == 0:
                raise StepError(f"request {e.rid!r} brings no tokens")
            bad = [t for t in e.tokens if not (0 <= int(t) < self.vocab_size)]
            if bad:
                raise StepError(f"request {e.rid!r}: token ids {bad[:8]} outside [0, {self.vocab_size})")
            if self.manager.length(e.rid) + n > self.max_position:
                raise StepError(f"request {e.rid!r}: {self.manager.length(e.rid)} + {n} tokens exceed max_position {self.max_position}")
            badw = [w for w in e.want if not (0 <= int(w) < n)]
            if badw:
                raise StepError(f"request {e.rid!r}: wanted places {badw[:8]} outside its {n} tokens")

    def prepare_decode(self, rids: Sequence[Hashable]) -> bool:
        """Get ready, while the GPU still works on the last step, everything that does not depend on the tokens of
        a step in which each of ``rids`` brings one token and wants its logits: checks, pages, the step's arrays.
        ``step`` uses it if that is the step it is given, and drops it otherwise (pages taken early stay with their
        request and are used or freed with it).  Returns False, having changed nothing, when it cannot (no graphs,
        a request at its last position, not enough pages)."""
        self._prepared = None
        rids = list(rids)
        if not self.decode_graphs or not rids or len(set(rids)) != len(rids):
            return False
        if not all(self.manager.has(r) and self.manager.length(r) + 1 <= self.max_position for r in rids):
            return False
        needs = [(r, 1) for r in rids]
        if not self.manager.can_reserve(needs):
            return False
        for r in rids:
            self.manager.reserve(r, 1)
        ctx = self._decode_context([StepEntry(r, [0], [0]) for r in rids])
        self._prepared = (self.manager.snapshot(rids), ctx)
        return True

    def _decode_context(self, entries) -> StepContext:
        """The context of a step of single tokens in the layout its captured graph has: block tables as wide as the
        next multiple of GRAPH_WIDTH_MULTIPLE pages, the batch filled up to the next of GRAPH_BATCH_SIZES."""
        n = len(entries)
        size = next((b for b in self.GRAPH_BATCH_SIZES if b >= n), -(-n // 16) * 16)
        return StepContext(entries, self.manager, self.dtype, self.device, width_multiple=self.GRAPH_WIDTH_MULTIPLE,
                           upload=False, pad_requests=size - n, scratch_pages=self.storage.scratch_pages,
                           scratch_state_slot=self.storage.scratch_state_slot)

    @property
    def starts_steps_early(self) -> bool:
        """Whether ``launch_prepared`` can ever start a step (graphs are on and no mixer keeps state of its own)."""
        return self.decode_graphs and not self.storage.has_state

    def launch_prepared(self, tokens: torch.Tensor, host_tokens: Optional[torch.Tensor] = None) -> bool:
        """Start the step ``prepare_decode`` got ready, now, with its tokens taken on the GPU from ``tokens`` (int32,
        one per request of that step, in its order: the sampler's output for the step before), so that the GPU goes
        on while the host reads those tokens and does its bookkeeping.  ``step`` hands out the logits if it is then
        given these requests with one token each, the very tokens of ``tokens``, or a part of them in the same
        order (the others' rows are dropped: a request that has just stopped).  ``host_tokens`` is a host copy of
        ``tokens`` that is complete by the time ``step`` is called (the sampler's pinned one); without it a copy
        is made here.  Any other step, or other tokens, makes the early step void and is computed afresh; keys and values written early are written again, which is
        why nothing is started early for a model whose mixers keep state of their own.
        Returns False, the prepared step kept for ``step``, when it cannot (no captured graph of this layout yet)."""
        prep = self._prepared
        if prep is None or self.storage.has_state:
            return False
        snapshot, ctx = prep
        g = self._graphs.get(ctx.layout_key)
        if g is None or tokens.dtype != torch.int32 or tuple(tokens.shape) != (ctx.n_real_tokens,) or tokens.device != self.device:
            return False
        self._prepared = None
        self._replay_inputs(g, ctx)
        g.ctx.token_ids[:ctx.n_real_tokens].copy_(tokens)   # (the copy above brought placeholder tokens; both precede the graph on the stream)
        g.graph.replay()
        self.graph_replays += 1
        copied = None
        if host_tokens is None:
            host_tokens = torch.empty(tokens.shape, dtype=torch.int32, pin_memory=True).copy_(tokens, non_blocking=True)
            copied = torch.cuda.Event()
            copied.record()
        self._launched = (snapshot, g, host_tokens, copied)
        return True

    def _take_launched(self, entries):
        """The logits of the step started early, if ``entries`` are its requests or a part of them; else None."""
        (snapshot, g, host_tokens, copied), self._launched = self._launched, None
        if any(len(e.tokens) != 1 or len(e.want) != 1 or e.want[0] != 0 for e in entries):
            return None
        if copied is not None:
            copied.synchronize()
        started_with = host_tokens.tolist()                 # the tokens the early step ran on
        rids, was = [e.rid for e in entries], snapshot[0]
        if len(rids) == len(was):
            if [int(e.tokens[0]) for e in entries] != started_with or not self.manager.unchanged(snapshot, rids):
                return None
            self.manager.commit_each(rids, 1)
            return g.logits[:len(rids)]
        place = {r: i for i, r in enumerate(was)}
        rows = [place.get(r, -1) for r in rids]
        if min(rows) < 0 or any(a >= b for a, b in zip(rows, rows[1:])):
            return None
        if [int(e.tokens[0]) for e in entries] != [started_with[i] for i in rows]:
            return None
        if not self.manager.unchanged(self.manager.snapshot_rows(snapshot, rows), rids):
            return None
        self.manager.commit_each(rids, 1)
        return ops.embedding(torch.tensor(rows, dtype=torch.int32, device=self.device), g.logits)    # those rows of the logits

    def _replay_inputs(self, g, ctx) -> None:
        g.copied.synchronize()          # the host buffer is free again once the last copy out of it is done
        ctx.write_host(g.host)          # (the replay reads the graph's own views of the slab: none are made here)
        g.slab.copy_(g.pinned, non_blocking=True)
        g.copied.record()

    def _take_prepared(self, entries):
        """The context ``prepare_decode`` built, if ``entries`` are the step it was built for (the same live
        requests, none of which has moved since), with their tokens put in; else None."""
        prep, self._prepared = self._prepared, None
        if prep is None or any(len(e.tokens) != 1 or len(e.want) != 1 or e.want[0] != 0 for e in entries):
            return None
        if not self.manager.unchanged(prep[0], [e.rid for e in entries]):
            return None
        tokens = [int(e.tokens[0]) for e in entries]
        if min(tokens) < 0 or max(tokens) >= self.vocab_size:
            return None                      # the full check names the culprit
        prep[1].set_tokens(entries, tokens)
        return prep[1]

    def step(self, entries: Sequence[StepEntry]) -> torch.Tensor:
        entries = list(entries)
        if not entries:
            return torch.empty((0, self.vocab_size), dtype=torch.float32, device=self.device)
        if self._launched is not None:
            logits = self._take_launched(entries)
            if logits is not None:
                return logits
        ctx = self._take_prepared(entries) if self._prepared is not None else None
        if ctx is not None:
            logits = self._decode_step(entries, ctx)
            self.manager.commit_each([e.rid for e in entries], 1)
            return logits
        self.validate(entries)
        needs = [(e.rid, len(e.tokens)) for e in entries]
        if not self.manager.can_reserve(needs):
            tot = [0] * len(self.manager.groups)
            for rid, n in needs:
                for g, k in enumerate(self.manager.pages_needed(rid, n)):
                    tot[g] += k
            g = next(g for g, t in enumerate(tot) if t > self.manager.pools[g].num_free)
            raise OutOfPages(g, tot[g], self.manager.pools[g].num_free)
        for rid, n in needs:
            self.manager.reserve(rid, n)
        if self.decode_graphs and all(n == 1 for _, n in needs):
            logits = self._decode_step(entries)
        else:
            ctx = StepContext(entries, self.manager, self.dtype, self.device)
            ctx.timer = self.timer
            logits = self.model.forward(ctx, self.storage)
        for rid, n in needs:
            self.manager.commit(rid, n)
        return logits

    def _decode_step(self, entries, ctx=None) -> torch.Tensor:
        """A step of single tokens through a captured graph.  The first step of a layout runs as usual
        and is then captured; later steps copy their arrays into the graph's buffer and replay it.
        The logits returned by a replay live in the graph's memory: they are valid until the next step."""
        if ctx is None:
            ctx = self._decode_context(entries)
        n = ctx.n_real_logit_rows
        g = self._graphs.get(ctx.layout_key)
        if g is not None:
            self._graphs[ctx.layout_key] = self._graphs.pop(ctx.layout_key)      # used last: evicted last
            self._replay_inputs(g, ctx)
            g.graph.replay()
            self.graph_replays += 1
            return g.logits[:n]
        slab = torch.empty(ctx.slab_size, dtype=torch.int32, device=self.device)
        pinned = torch.empty(ctx.slab_size, dtype=torch.int32, pin_memory=True)
        ctx.bind(slab, pinned)
        logits = self.model.forward(ctx, self.storage)            # this step, eagerly (also loads every kernel)
        if len(self._graphs) >= self.MAX_GRAPHS:
            self._graphs.pop(next(iter(self._graphs)))
        torch.cuda.synchronize()
        cap_ctx = self._decode_context(entries)
        cap_ctx.use_slab(slab)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            cap_logits = self.model.forward(cap_ctx, self.storage)
        self._graphs[ctx.layout_key] = _DecodeGraph(slab, pinned, graph, cap_ctx, cap_logits)
        self.graph_captures += 1
        return logits[:n]
