"""Per-request sampling parameters, with the reference's names, defaults and meanings
(scheduler/request_batch.h:26-38): temperature (0 = greedy), top_p (1.0 = off), top_k (0 = off),
min_p (0 = off), frequency_penalty, presence_penalty, repetition_penalty (1.0 = off),
penalty_last_n (64), seed (UINT32_MAX = a fresh seed per request), logit_bias.

Differences from the reference's native sampler, which are deliberate: top_k, min_p and
logit_bias are honoured (it ignores them, runtime/backends/cuda/native/gpu_sampler.cu:563-567);
a greedy request gets no implicit repetition penalty of 1.15
(runtime/backends/cuda/inferflux_cuda_executor.cpp:3367-3371); and a seeded request draws a new
uniform number at every step, u = philox(seed, step), instead of re-seeding the generator before
each draw, which repeats the same number (gpu_sampler.cu:603-605).
"""
from __future__ import annotations

import dataclasses
import os
from typing import Dict, Optional, Sequence

import numpy as np

UNSEEDED = 0xFFFFFFFF


@dataclasses.dataclass
class SamplingParams:
    temperature: float = 1.0
    top_p: float = 1.0
    top_k: int = 0
    min_p: float = 0.0
    frequency_penalty: float = 0.0
    presence_penalty: float = 0.0
    repetition_penalty: float = 1.0
    penalty_last_n: int = 64
    seed: int = UNSEEDED
    logit_bias: Dict[int, float] = dataclasses.field(default_factory=dict)
    max_tokens: int = 16
    stop_token_ids: Sequence[int] = ()
    ignore_eos: bool = False
    # None: no log-probabilities; 0: the sampled token's; N (at most 20): with the N most probable
    # alternatives (the reference's collect_logprobs / logprob_top_n, scheduler/request_batch.h:258-265)
    logprobs: Optional[int] = None

    def validate(self) -> None:
        if self.temperature < 0:
            raise ValueError("temperature must be >= 0 (0 = greedy)")
        if not (0.0 < self.top_p <= 1.0):
            raise ValueError("top_p must be in (0, 1]")
        if self.top_k < 0 or not (0.0 <= self.min_p <= 1.0):
            raise ValueError("top_k must be >= 0 and min_p in [0, 1]")
        if self.repetition_penalty <= 0:
            raise ValueError("repetition_penalty must be positive (1.0 = off)")
        if self.penalty_last_n < 0 or self.max_tokens < 1:
            raise ValueError("penalty_last_n must be >= 0 and max_tokens >= 1")
        if self.logprobs is not None and not (0 <= self.logprobs <= 20):
            raise ValueError("logprobs must be None or between 0 and 20")
        if not (0 <= int(self.seed) < 1 << 64):
            raise ValueError("seed must be a non-negative number of at most 64 bits")

    @property
    def greedy(self) -> bool:
        return self.temperature <= 0.0

    @property
    def has_penalties(self) -> bool:
        return self.repetition_penalty != 1.0 or self.frequency_penalty != 0.0 or self.presence_penalty != 0.0


def fresh_seed() -> int:
    return int.from_bytes(os.urandom(4), "little") % UNSEEDED


_M0, _M1 = np.uint64(0xD2511F53), np.uint64(0xCD9E8D57)
_W0, _W1 = np.uint32(0x9E3779B9), np.uint32(0xBB67AE85)
_MASK = np.uint64(0xFFFFFFFF)


def philox4x32_10(counter, key):
    """The ten rounds of Philox4x32 (Salmon et al., "Parallel random numbers: as easy as 1, 2, 3", 2011) on arrays:
    ``counter`` four and ``key`` two arrays of 32-bit words (as uint64); returns the four output words."""
    c = [np.asarray(w, dtype=np.uint64) & _MASK for w in counter]
    k0, k1 = (np.asarray(key[0], dtype=np.uint64) & _MASK).astype(np.uint32), (np.asarray(key[1], dtype=np.uint64) & _MASK).astype(np.uint32)
    with np.errstate(over="ignore"):
        for _ in range(10):
            p0, p1 = _M0 * c[0], _M1 * c[2]
            c = [((p1 >> np.uint64(32)) ^ c[1] ^ k0.astype(np.uint64)) & _MASK, p1 & _MASK,
                 ((p0 >> np.uint64(32)) ^ c[3] ^ k1.astype(np.uint64)) & _MASK, p0 & _MASK]
            k0, k1 = k0 + _W0, k1 + _W1
    return c


def philox_uniform(seeds: np.ndarray, steps: np.ndarray) -> np.ndarray:
    """One float32 in [0, 1) per (seed, step): Philox4x32-10 keyed by the seed, counter = step; the top 24 bits of
    the first output word.

    A counter-based generator: the number depends on the pair alone, not on what was drawn before
    or on which other requests share the batch (the reference's invariant that batched sampling
    with per-sequence seeds equals single-sequence sampling, tests/unit/test_gpu_sampler.cpp:205-262).
    """
    seeds = np.asarray(seeds, dtype=np.uint64)
    steps = np.asarray(steps, dtype=np.uint64)
    zero = np.zeros_like(steps)
    c = philox4x32_10([steps & _MASK, steps >> np.uint64(32), zero, zero], [seeds & _MASK, seeds >> np.uint64(32)])
    return ((c[0] >> np.uint64(8)).astype(np.float64) * (1.0 / (1 << 24))).astype(np.float32)
