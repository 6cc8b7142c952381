"""Turns a step's logits into tokens: penalties and logit bias, then argmax or a seeded draw.

All arithmetic on the logits is done by the HIP kernels (kernels.ops); this module gathers each
request's parameters and history into flat arrays.  Order, as in the reference
(runtime/backends/cuda/inferflux_cuda_executor.cpp:3363-3402): penalties over the request's last
``penalty_last_n`` sampled tokens, then sampling.
"""
from __future__ import annotations

import dataclasses
from typing import List, Sequence

import numpy as np
import torch

from ..kernels import ops
from .params import UNSEEDED, SamplingParams, fresh_seed


@dataclasses.dataclass
class TokenLogprob:
    """The sampled token's log-probability (log-softmax of the logits after penalties and bias, before
    temperature) and the most probable alternatives [(token id, log-probability)], as the reference
    reports them (runtime/logprob.h:11-18; token ids here, the engine has no text)."""
    token_id: int
    logprob: float
    top_logprobs: List = dataclasses.field(default_factory=list)


@dataclasses.dataclass
class SamplingState:
    """What sampling remembers of a request between steps."""
    params: SamplingParams
    seed: int = 0
    draws: int = 0                      # stochastic draws so far: the generator's counter
    history: List[int] = dataclasses.field(default_factory=list)   # the last penalty_last_n sampled tokens, oldest first
    seen: dict = dataclasses.field(default_factory=dict)            # token -> how often it occurs in ``history``
    logprobs: List[TokenLogprob] = dataclasses.field(default_factory=list)

    @classmethod
    def start(cls, params: SamplingParams) -> "SamplingState":
        params.validate()
        return cls(params, seed=fresh_seed() if params.seed == UNSEEDED else int(params.seed))

    def record(self, token: int) -> None:
        n = self.params.penalty_last_n
        if not n:
            return
        token = int(token)
        self.history.append(token)
        self.seen[token] = self.seen.get(token, 0) + 1
        while len(self.history) > n:
            old = self.history.pop(0)
            left = self.seen[old] - 1
            if left:
                self.seen[old] = left
            else:
                del self.seen[old]


class Sampler:
    def __init__(self, device):
        self.device = device
        self._host_results = {}       # pinned: the chosen tokens and their log-probabilities come to the host through these
        self._host_words = None       # pinned: a step's parameters go to the GPU through it
        self._host_used = 0           # words of it that this step's copies are reading
        self._copied = torch.cuda.Event()

    def _to_host(self, t: torch.Tensor, name: str) -> torch.Tensor:
        """An asynchronous copy of ``t`` into pinned host memory kept under ``name`` and used again by the next step
        (valid once ``_copied`` has been waited for, until the next call with that name)."""
        held = self._host_results.get(name)
        if held is None or held.dtype != t.dtype or held.shape[0] < t.numel():
            held = self._host_results[name] = torch.empty(max(64, 2 * t.numel()), dtype=t.dtype, pin_memory=True)
        return held[:t.numel()].view(t.shape).copy_(t, non_blocking=True)

    def _upload(self, *arrays):
        """Lists or 1-D arrays of int32 or float32 numbers as GPU tensors, through pinned memory in one copy.  The pinned
        words are reused by the next step: ``sample`` waits for its copies before it returns."""
        arrays = [np.ascontiguousarray(a, dtype=np.float32 if np.asarray(a).dtype.kind == "f" else np.int32) for a in arrays]
        total = sum(a.shape[0] for a in arrays)
        if self._host_words is None or self._host_words.shape[0] < self._host_used + total:
            self._host_words = torch.empty(max(4096, 2 * (self._host_used + total)), dtype=torch.int32, pin_memory=True)
            self._host_used = 0       # the old words stay alive until their copies are done: torch keeps them
        host = self._host_words[self._host_used: self._host_used + total]
        self._host_used += total
        words, at = host.numpy(), 0
        for a in arrays:
            words[at: at + a.shape[0]] = a.view(np.int32)
            at += a.shape[0]
        dev = torch.empty(total, dtype=torch.int32, device=self.device).copy_(host, non_blocking=True)
        out, at = [], 0
        for a in arrays:
            t = dev[at: at + a.shape[0]]
            out.append(t.view(torch.float32) if a.dtype == np.float32 else t)
            at += a.shape[0]
        return out

    def sample(self, logits: torch.Tensor, states: Sequence[SamplingState], while_waiting=None) -> List[int]:
        """One token per row of float32 ``logits`` [R, V]; row i belongs to ``states[i]``.  The
        logits are modified in place by penalties and bias.  States are advanced (draw counter,
        history).  ``while_waiting`` is called with the chosen tokens (int32 [R], on the GPU) and the pinned host
        tensor their copy is on its way to (valid once this function has returned) once the kernels and
        the copies of their results to the host are launched, before these are waited for: host work that needs no
        token goes there, and so may GPU work that takes the tokens where they are; the wait is for the copies
        only, not for what ``while_waiting`` launched."""
        R = logits.shape[0]
        if R != len(states):
            raise ValueError(f"{R} rows of logits for {len(states)} requests")
        if R == 0:
            return []
        self._host_used = 0
        rows, ids, counts = [], [], []
        brow, bid, bval = [], [], []
        for r, st in enumerate(states):
            p = st.params
            if p.has_penalties and p.penalty_last_n > 0 and st.history:
                rows += [r] * len(st.seen); ids += st.seen.keys(); counts += st.seen.values()
            for t, b in p.logit_bias.items():
                brow.append(r); bid.append(int(t)); bval.append(float(b))
        if rows:
            ops.apply_penalties(logits, *self._upload(
                np.asarray(rows, np.int32), np.asarray(ids, np.int32), np.asarray(counts, np.int32),
                np.asarray([s.params.repetition_penalty for s in states], np.float32),
                np.asarray([s.params.frequency_penalty for s in states], np.float32),
                np.asarray([s.params.presence_penalty for s in states], np.float32)))
        if brow:
            ops.add_logit_bias(logits, *self._upload(np.asarray(brow, np.int32), np.asarray(bid, np.int32),
                                                     np.asarray(bval, np.float32)))
        if all(s.params.greedy for s in states):
            chosen = ops.argmax(logits)
        else:
            # the kernel makes each row's number in [0, 1) itself, as params.philox_uniform does, from (seed, draws so far)
            pairs = np.array([[s.seed, s.draws] for s in states], dtype=np.uint64)
            words = np.ascontiguousarray(pairs).view(np.uint32).view(np.int32).reshape(-1)    # low word first
            temperature, top_k, top_p, min_p, draws = self._upload(
                np.asarray([s.params.temperature for s in states], np.float32),
                np.asarray([s.params.top_k for s in states], np.int32),
                np.asarray([s.params.top_p for s in states], np.float32),
                np.asarray([s.params.min_p for s in states], np.float32), words)
            chosen = ops.sample(logits, temperature, top_k, top_p, min_p, draws=draws.view(R, 4),
                                any_greedy=any(s.params.greedy for s in states),
                                any_filters=any(s.params.top_k > 0 or s.params.top_p < 1.0 for s in states))
        top_n = max((s.params.logprobs for s in states if s.params.logprobs is not None), default=None)
        if top_n is not None:
            lp_dev = ops.logprobs(logits, chosen, top_n)
            lp, top_ids, top_lp = (self._to_host(t, name) for t, name in zip(lp_dev, ("lp", "top_ids", "top_lp")))
        host_tokens = self._to_host(chosen, "tokens")
        self._copied.record()
        if while_waiting is not None:
            while_waiting(chosen, host_tokens)
        self._copied.synchronize()
        tokens = host_tokens.tolist()
        if top_n is not None:
            lp, top_ids, top_lp = lp.tolist(), top_ids.tolist(), top_lp.tolist()
            for r, (st, t) in enumerate(zip(states, tokens)):
                if st.params.logprobs is not None:
                    n = st.params.logprobs
                    st.logprobs.append(TokenLogprob(int(t), lp[r], list(zip(top_ids[r][:n], top_lp[r][:n]))))
        for st, t in zip(states, tokens):
            if not st.params.greedy:
                st.draws += 1
            st.record(t)
        return tokens
