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
from .params import UNSEEDED, SamplingParams, fresh_seed, philox_uniform


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
    history: List[int] = dataclasses.field(default_factory=list)   # sampled tokens, oldest first
    logprobs: List[TokenLogprob] = dataclasses.field(default_factory=list)

    @classmethod
    def start(cls, params: SamplingParams) -> "SamplingState":
        params.validate()
        return cls(params, seed=fresh_seed() if params.seed == UNSEEDED else int(params.seed))

    def record(self, token: int) -> None:
        self.history.append(int(token))
        n = self.params.penalty_last_n
        if n and len(self.history) > n:
            del self.history[: len(self.history) - n]


class Sampler:
    def __init__(self, device):
        self.device = device
        self._host_tokens = None      # pinned: the chosen tokens come to the host through it
        self._copied = torch.cuda.Event()

    def _to_host(self, t: torch.Tensor, keep: bool = False) -> torch.Tensor:
        """An asynchronous copy of ``t`` into pinned host memory (valid once ``_copied`` has been waited for)."""
        if keep:
            if self._host_tokens is None or self._host_tokens.shape[0] < t.shape[0]:
                self._host_tokens = torch.empty(max(64, t.shape[0]), dtype=t.dtype, pin_memory=True)
            out = self._host_tokens[:t.shape[0]]
        else:
            out = torch.empty(t.shape, dtype=t.dtype, pin_memory=True)
        return out.copy_(t, non_blocking=True)

    def _dev(self, values, dtype):
        return torch.tensor(values, dtype=dtype, device=self.device)

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
        rows, ids, counts = [], [], []
        brow, bid, bval = [], [], []
        for r, st in enumerate(states):
            p = st.params
            if p.has_penalties and p.penalty_last_n > 0 and st.history:
                uniq, cnt = np.unique(np.asarray(st.history[-p.penalty_last_n:], dtype=np.int64), return_counts=True)
                rows += [r] * len(uniq); ids += uniq.tolist(); counts += cnt.tolist()
            for t, b in p.logit_bias.items():
                brow.append(r); bid.append(int(t)); bval.append(float(b))
        if rows:
            ops.apply_penalties(logits, self._dev(rows, torch.int32), self._dev(ids, torch.int32),
                                self._dev(counts, torch.int32),
                                self._dev([s.params.repetition_penalty for s in states], torch.float32),
                                self._dev([s.params.frequency_penalty for s in states], torch.float32),
                                self._dev([s.params.presence_penalty for s in states], torch.float32))
        if brow:
            ops.add_logit_bias(logits, self._dev(brow, torch.int32), self._dev(bid, torch.int32), self._dev(bval, torch.float32))
        if all(s.params.greedy for s in states):
            chosen = ops.argmax(logits)
        else:
            u = philox_uniform(np.array([s.seed for s in states]), np.array([s.draws for s in states]))
            chosen = ops.sample(logits,
                                self._dev([s.params.temperature for s in states], torch.float32),
                                self._dev([s.params.top_k for s in states], torch.int32),
                                self._dev([s.params.top_p for s in states], torch.float32),
                                self._dev([s.params.min_p for s in states], torch.float32),
                                torch.from_numpy(u).to(self.device))
        top_n = max((s.params.logprobs for s in states if s.params.logprobs is not None), default=None)
        if top_n is not None:
            lp_dev = ops.logprobs(logits, chosen, top_n)
            lp, top_ids, top_lp = (self._to_host(t) for t in lp_dev)
        host_tokens = self._to_host(chosen, keep=True)
        self._copied.record()
        if while_waiting is not None:
            while_waiting(chosen, host_tokens)
        self._copied.synchronize()
        tokens = host_tokens.tolist()
        for r, (st, t) in enumerate(zip(states, tokens)):
            if st.params.logprobs is not None:
                n = st.params.logprobs
                st.logprobs.append(TokenLogprob(int(t), float(lp[r]),
                                                list(zip(top_ids[r, :n].tolist(), top_lp[r, :n].tolist()))))
        for st, t in zip(states, tokens):
            if not st.params.greedy:
                st.draws += 1
            st.record(t)
        return tokens
