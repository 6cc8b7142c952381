"""The engine: requests in, tokens out.  Scheduler above, step function below, sampler beside.

Programming interface in the shape of the reference's runtime (LoadModel / ExecuteUnifiedBatch /
NativeFreeSequence / Generate: runtime/backends/native/native_inference_runtime.h:34-37, 91):
``Engine.load`` (a model folder), ``add_request``, ``step`` (one scheduled step; returns what
finished), ``abort``, ``generate`` (run a list of prompts to completion), ``stats`` (the
reference's perf snapshot {prefill_ms, decode_ms, prompt_tokens, generated_tokens},
native_inference_runtime.h:58-64).  Prompts are token ids; text is outside the engine.
"""
from __future__ import annotations

import dataclasses
import time
from typing import Callable, Dict, Hashable, List, Optional, Sequence

from .. import log
from ..sampling.params import SamplingParams
from ..sampling.sampler import Sampler, SamplingState
from .api import load_runner
from .load_spec import ModelLoadSpec
from .context import StepEntry
from .runner import ModelRunner
from .scheduler import RequestRefused, Scheduler, SchedulerConfig, Sequence_


@dataclasses.dataclass
class RequestOutput:
    request_id: Hashable
    prompt_token_ids: List[int]
    token_ids: List[int]
    finish_reason: Optional[str] = None      # "stop" (eos or a stop token), "length", "abort"; None while running
    preemptions: int = 0
    logprobs: Optional[List] = None          # one sampler.TokenLogprob per generated token, when asked for

    @property
    def finished(self) -> bool:
        return self.finish_reason is not None


@dataclasses.dataclass
class EngineStats:
    prefill_ms: float = 0.0
    decode_ms: float = 0.0
    prompt_tokens: int = 0
    generated_tokens: int = 0
    steps: int = 0
    preemptions: int = 0
    # steps by their number of tokens: key 2**k counts the steps of more than 2**(k-1) and at most 2**k tokens
    step_tokens: Dict[int, int] = dataclasses.field(default_factory=dict)


class _Live:
    def __init__(self, seq: Sequence_, params: SamplingParams, prompt: List[int]):
        self.seq, self.params, self.prompt = seq, params, prompt
        self.sampling = SamplingState.start(params)


def quiet_garbage_collector() -> None:
    """For a process that is about to serve: collect once, then move everything alive now (the interpreter's and the
    libraries' millions of objects, the loaded model) out of the collector's sight.  A full collection walks all of them
    (tens of milliseconds with torch imported) and comes every few hundred steps of a busy engine otherwise.  What
    is alive now is then only freed by reference counts, so this is for the entry points to call, not the library."""
    import gc
    gc.collect()
    gc.freeze()


class Engine:
    def __init__(self, runner: ModelRunner, scheduler_config: Optional[SchedulerConfig] = None,
                 start_steps_early: bool = True):
        self.runner = runner
        self.start_steps_early = start_steps_early   # decode steps are started before the host has read the last step's tokens
        self.config = scheduler_config or SchedulerConfig()
        self.config.max_batch_size = min(self.config.max_batch_size, runner.manager.max_requests)
        self.scheduler = Scheduler(runner.manager, self.config, runner.max_position)
        self.sampler = Sampler(runner.device)
        self.eos_token_ids = frozenset(runner.model.plan.eos_token_ids)
        self._live: Dict[Hashable, _Live] = {}
        self._next_id = 0
        self.stats = EngineStats()

    @classmethod
    def load(cls, model, dtype: str = "bfloat16", kv_pages: Optional[int] = None, page_size: int = 16,
             max_batch_size: int = 32, max_batch_tokens: int = 16384, chunked_prefill_tokens: int = 512,
             ctx_size: int = 4096, phase_timing: bool = False, decode_weight_copy: bool = True,
             start_steps_early: bool = True, library_gemm_tuning: bool = False,
             prefill_tokens_alone: Optional[int] = None) -> "Engine":
        """``model`` is a ``ModelLoadSpec``, or a model folder with the other arguments standing for the spec's
        fields (``max_batch_size`` = max_parallel_sequences, ``ctx_size`` = context_size).  ``kv_pages`` None sizes
        the cache for ``ctx_size`` tokens for each of ``max_batch_size`` requests, within the device memory that is
        free once the weights are loaded.  ``decode_weight_copy`` False saves the second, tiled copy of the weights
        at the price of slower decoding.  ``prefill_tokens_alone``: the largest portion of a prompt in a step in which
        nobody decodes (None: 2,048, or ``chunked_prefill_tokens`` if that is more).  ``library_gemm_tuning`` lets the library time its kernels for the product shapes
        of prompts (see ``ops.enable_library_gemm_tuning``)."""
        spec = model if isinstance(model, ModelLoadSpec) else ModelLoadSpec(
            path=model, dtype=dtype, kv_pages=kv_pages, page_size=page_size, max_parallel_sequences=max_batch_size,
            max_batch_tokens=max_batch_tokens, chunked_prefill_tokens=chunked_prefill_tokens, context_size=ctx_size,
            phase_timing=phase_timing, decode_weight_copy=decode_weight_copy, library_gemm_tuning=library_gemm_tuning,
            prefill_tokens_alone=prefill_tokens_alone)
        runner = load_runner(spec.checked())
        log.info("engine", "model loaded", model=spec.path or spec.random_weights, dtype=spec.dtype,
                 kv_pages=runner.manager.pools[0].num_pages if runner.manager.pools else 0, page_size=spec.page_size,
                 max_batch_size=spec.max_parallel_sequences)
        return cls(runner, SchedulerConfig(spec.max_parallel_sequences, spec.max_batch_tokens, spec.chunked_prefill_tokens,
                                           spec.prefill_tokens_alone), start_steps_early)

    # ---- requests -----------------------------------------------------------------
    def add_request(self, prompt_token_ids: Sequence[int], params: Optional[SamplingParams] = None,
                    request_id: Optional[Hashable] = None, priority: int = 0) -> Hashable:
        """Queue a request; it joins the running batch at the next ``step`` that has room for it.  ``priority``:
        higher is admitted earlier and preempted later (equal priorities: first come first served)."""
        params = params or SamplingParams()
        params.validate()
        prompt = [int(t) for t in prompt_token_ids]
        bad = [t for t in prompt if not (0 <= t < self.runner.vocab_size)]
        if bad:
            raise RequestRefused(f"token ids {bad[:8]} outside [0, {self.runner.vocab_size})")
        if request_id is None:
            request_id = self._next_id
            self._next_id += 1
        seq = self.scheduler.add(request_id, prompt, params.max_tokens, priority)
        self._live[request_id] = _Live(seq, params, prompt)
        self.stats.prompt_tokens += len(prompt)
        return request_id

    def abort(self, request_id: Hashable) -> Optional[RequestOutput]:
        live = self._live.pop(request_id, None)
        if live is None:
            return None
        self.scheduler.finish(live.seq)
        return RequestOutput(request_id, live.prompt, list(live.seq.generated), "abort", live.seq.preemptions)

    def has_unfinished(self) -> bool:
        return self.scheduler.has_work()

    # ---- one step -------------------------------------------------------------------
    def _finish_reason(self, live: _Live, token: int) -> Optional[str]:
        p = live.params
        if not p.ignore_eos and token in self.eos_token_ids:
            return "stop"
        if token in p.stop_token_ids:
            return "stop"
        if len(live.seq.generated) >= p.max_tokens:
            return "length"
        return None

    def step(self, on_token: Optional[Callable[[Hashable, int], None]] = None) -> List[RequestOutput]:
        """Run one scheduled step; returns the requests that finished in it."""
        plan = self.scheduler.schedule()
        self.stats.preemptions += len(plan.preempted)
        if not plan.items:
            if self.scheduler.has_work():
                raise RuntimeError("the scheduler has work but could plan nothing (pool too small for any request?)")
            return []
        t0 = time.perf_counter()
        entries = [StepEntry(i.seq.rid, i.tokens, [len(i.tokens) - 1] if i.wants_logits else []) for i in plan.items]
        logits = self.runner.step(entries)
        wanting = [i for i in plan.items if i.wants_logits]
        ahead = None
        if len(wanting) == len(plan.items) and not self.scheduler.waiting and all(len(i.tokens) == 1 for i in plan.items):
            # A step of decoding with nobody waiting: the next step is most likely the same requests, one token
            # further, less those that reach their limit now.  While the GPU works on this one, the runner gets
            # ready what of the next does not depend on its tokens; if the guess is wrong it is dropped.
            # Where it can, the runner also starts that step, for everyone of this one and with the tokens taken on
            # the GPU: the host then reads them and does its bookkeeping while the GPU is already at work on the
            # next step.  A request that is at its limit, or stops on a token nobody could foresee, only has its
            # row of that step dropped.
            everyone = [i.seq.rid for i in plan.items]
            staying = [i.seq.rid for i in plan.items if len(i.seq.generated) + 1 < self._live[i.seq.rid].params.max_tokens]
            early = self.start_steps_early and self.runner.starts_steps_early and bool(staying)

            def ahead(chosen, host_tokens):
                if early:
                    if self.runner.prepare_decode(everyone) and self.runner.launch_prepared(chosen, host_tokens):
                        return
                    if len(staying) == len(everyone):
                        return                      # what was got ready stands
                self.runner.prepare_decode(staying)
        tokens = self.sampler.sample(logits, [self._live[i.seq.rid].sampling for i in wanting], ahead) if wanting else []
        dt = (time.perf_counter() - t0) * 1e3
        if any(len(i.tokens) > 1 or i.seq.is_prefilling for i in plan.items):
            self.stats.prefill_ms += dt
        else:
            self.stats.decode_ms += dt
        self.stats.steps += 1
        bucket = 1 << (sum(len(i.tokens) for i in plan.items) - 1).bit_length()
        self.stats.step_tokens[bucket] = self.stats.step_tokens.get(bucket, 0) + 1
        for i in plan.items:
            self.scheduler.advance(i)
        done: List[RequestOutput] = []
        for i, tok in zip(wanting, tokens):
            live = self._live[i.seq.rid]
            i.seq.generated.append(int(tok))
            self.stats.generated_tokens += 1
            if on_token is not None:
                on_token(i.seq.rid, int(tok))
            reason = self._finish_reason(live, int(tok))
            if reason is not None:
                self.scheduler.finish(i.seq)
                del self._live[i.seq.rid]
                done.append(RequestOutput(i.seq.rid, live.prompt, list(i.seq.generated), reason, i.seq.preemptions,
                                          list(live.sampling.logprobs) if live.params.logprobs is not None else None))
        return done

    def generate(self, prompts: Sequence[Sequence[int]], params=None,
                 on_token: Optional[Callable[[Hashable, int], None]] = None) -> List[RequestOutput]:
        """Run ``prompts`` (lists of token ids) to completion; results in the order of the prompts.
        ``params`` is one SamplingParams for all or one per prompt."""
        if params is None or isinstance(params, SamplingParams):
            params = [dataclasses.replace(params) if params else SamplingParams() for _ in prompts]
        ids = [self.add_request(p, sp) for p, sp in zip(prompts, params)]
        results: Dict[Hashable, RequestOutput] = {}
        while any(i not in results for i in ids):
            for out in self.step(on_token):
                results[out.request_id] = out
        return [results[i] for i in ids]
