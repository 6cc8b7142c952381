"""Generation through the entry points: greedy tokens against the plain implementation, sampling
with a seed against the plain rule, preemption by recomputation, and the command line."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_model as pm
from conftest import ROOT, TINY, seeded_ids

pytestmark = pytest.mark.gpu

if torch.cuda.is_available():
    from inferflux_amd import Engine, SamplingParams
    from inferflux_amd.sampling.params import philox_uniform

# Generation workloads of the tiny configurations: prompts of 7/13/29 tokens with 16 greedy tokens
# each (A); prompts of 1/17/64/100/250 with 24 tokens, prefill portions of 32, pages of 16 (B).
WORKLOADS = {"A": ([7, 13, 29], 16, 512), "B": ([1, 17, 64, 100, 250], 24, 32), "C": ([40, 3, 90], 20, 16)}


def plain_greedy(folder, prompt, n):
    cfg, W = pm.load_folder(folder, torch.float64)
    return pm.greedy_generate(cfg, W, prompt, n)


@pytest.mark.parametrize("name", list(TINY))
def test_greedy_generation_equals_the_plain_model(name, model_folders):
    folder = model_folders[name]
    lens, n_new, chunk = WORKLOADS[name]
    prompts = [seeded_ids(50 + i, n, TINY[name]["vocab_size"]) for i, n in enumerate(lens)]
    engine = Engine.load(folder, dtype="float32", kv_pages=64, max_batch_size=8, chunked_prefill_tokens=chunk,
                         prefill_tokens_alone=chunk)
    outs = engine.generate(prompts, SamplingParams(temperature=0.0, max_tokens=n_new, ignore_eos=True))
    for p, o in zip(prompts, outs):
        assert o.finish_reason == "length" and o.token_ids == plain_greedy(folder, p, n_new)
    assert engine.runner.manager.free_pages() == [64] * len(engine.runner.manager.groups)
    st = engine.stats
    assert st.generated_tokens == n_new * len(prompts) and st.prompt_tokens == sum(lens)


def test_steps_got_ready_and_started_ahead_change_no_token_and_are_used(model_folders, monkeypatch):
    """While the GPU decodes, the engine gets the next decode step ready on a guess (the same requests, less those at
    their limit) and, where nobody is at a limit, starts it with the tokens taken on the GPU.  A stop token makes the
    guess wrong once: only that request's row is dropped.  Tokens are the same with and without all this."""
    from inferflux_amd.engine.runner import ModelRunner
    folder = model_folders["B"]
    prompts = [seeded_ids(80 + i, n, TINY["B"]["vocab_size"]) for i, n in enumerate([5, 40, 23])]
    limits = (6, 30, 17)

    def run(stop, **kw):
        params = [SamplingParams(temperature=0.0, max_tokens=n, ignore_eos=True, stop_token_ids=stop if i == 1 else ())
                  for i, n in enumerate(limits)]
        eng = Engine.load(folder, dtype="bfloat16", kv_pages=64, max_batch_size=4, **kw)
        outs = eng.generate(prompts, params)
        eng.runner.manager.check()
        assert eng.runner.manager.free_pages() == [64]
        return outs

    taken, started = [], []
    real, real_launched = ModelRunner._take_prepared, ModelRunner._take_launched
    monkeypatch.setattr(ModelRunner, "_take_prepared", lambda self, e: _count(taken, real(self, e)))
    monkeypatch.setattr(ModelRunner, "_take_launched", lambda self, e: _count(started, real_launched(self, e)))
    with_it = run(())
    assert [len(o.token_ids) for o in with_it] == list(limits)
    assert sum(started) >= 15 and all(started) and all(taken)     # requests that reach their limit are foreseen
    n_taken = len(taken)
    ids1 = with_it[1].token_ids
    at = next(j for j in range(8, 16) if ids1[j] not in ids1[:j])   # a token's first appearance, while nobody is at a limit
    stop = [ids1[at]]
    del taken[:], started[:]
    stopped = run(stop)
    assert stopped[1].finish_reason == "stop" and stopped[1].token_ids == ids1[:at + 1]
    assert all(started) and all(taken)                             # the stopped request's row was dropped, no step lost
    del taken[:], started[:]
    only_ready = run((), start_steps_early=False)
    assert not started and len(taken) > n_taken and all(taken)
    assert [o.token_ids for o in only_ready] == [o.token_ids for o in with_it]
    assert [o.token_ids for o in run(stop, start_steps_early=False)] == [o.token_ids for o in stopped]
    monkeypatch.setattr(ModelRunner, "prepare_decode", lambda self, rids: False)
    assert [o.token_ids for o in run(())] == [o.token_ids for o in with_it]
    assert [o.token_ids for o in run(stop)] == [o.token_ids for o in stopped]


@pytest.mark.parametrize("seed", [0, 1])
def test_more_requests_than_slots_with_limits_stops_and_few_pages(seed, model_folders):
    """Requests come in as others finish, each with its own limit, some stopping on a token, with so few pages that
    some are preempted: in float32 every request's tokens are those of the plain model whether steps are started
    early or not (rows dropped from a step, steps made void by an arrival and computed afresh)."""
    folder, V = model_folders["C"], TINY["C"]["vocab_size"]
    rng = np.random.default_rng(seed)
    lens = rng.integers(2, 60, 14).tolist()
    limits = rng.integers(1, 28, 14).tolist()
    prompts = [seeded_ids(300 + 20 * seed + i, n, V) for i, n in enumerate(lens)]
    want = [plain_greedy(folder, p, n) for p, n in zip(prompts, limits)]
    stops = {i: [want[i][len(want[i]) // 2]] for i in range(0, 14, 3) if len(want[i]) > 3}    # stop half-way (or earlier)
    for i, st in stops.items():
        want[i] = want[i][: want[i].index(st[0]) + 1]

    def run(early, pages):
        eng = Engine.load(folder, dtype="float32", kv_pages=pages, max_batch_size=4, chunked_prefill_tokens=16,
                          prefill_tokens_alone=24, start_steps_early=early)
        params = [SamplingParams(temperature=0.0, max_tokens=n, ignore_eos=True, stop_token_ids=stops.get(i, ()))
                  for i, n in enumerate(limits)]
        outs = eng.generate(prompts, params)
        eng.runner.manager.check()
        assert eng.runner.manager.free_pages() == [pages] * len(eng.runner.manager.groups)
        return [o.token_ids for o in outs], eng.stats.preemptions

    for early in (True, False):
        got, _ = run(early, 64)
        assert got == want
    got, preempted = run(True, 9)                          # four requests of up to 87 tokens need up to 24 pages
    assert got == want and preempted >= 1


def _count(taken, ctx):
    taken.append(ctx is not None)
    return ctx


def test_preemption_by_recomputation_changes_no_token(model_folders):
    folder = model_folders["A"]
    prompts = [seeded_ids(70 + i, 40, 512) for i in range(3)]
    sp = SamplingParams(temperature=0.0, max_tokens=40, ignore_eos=True)
    roomy = Engine.load(folder, dtype="float32", kv_pages=64, max_batch_size=4)
    want = [o.token_ids for o in roomy.generate(prompts, sp)]
    tight = Engine.load(folder, dtype="float32", kv_pages=8, max_batch_size=4)     # 15 pages would be needed
    outs = tight.generate(prompts, sp)
    assert [o.token_ids for o in outs] == want
    assert tight.stats.preemptions >= 1 and outs[0].preemptions == 0
    tight.runner.manager.check()
    assert tight.runner.manager.free_pages() == [8]


def test_seeded_sampling_follows_the_plain_rule_and_ignores_batch_composition(model_folders):
    folder = model_folders["B"]
    cfg, W = pm.load_folder(folder, torch.float64)
    prompts = [seeded_ids(80 + i, n, 1000) for i, n in enumerate((5, 33, 12))]
    params = [SamplingParams(temperature=0.8, seed=11, max_tokens=24, ignore_eos=True),
              SamplingParams(temperature=1.0, top_p=0.9, top_k=50, seed=12, max_tokens=24, ignore_eos=True),
              SamplingParams(temperature=1.2, min_p=0.001, repetition_penalty=1.3, frequency_penalty=0.1,
                             presence_penalty=0.2, seed=13, max_tokens=24, ignore_eos=True)]
    engine = Engine.load(folder, dtype="float32", kv_pages=64, max_batch_size=4, chunked_prefill_tokens=32, prefill_tokens_alone=32)
    together = [o.token_ids for o in engine.generate(prompts, params)]
    alone = [engine.generate([p], [sp])[0].token_ids for p, sp in zip(prompts, params)]
    assert together == alone                                  # (seed, step) alone decides the draw
    assert len({tuple(t) for t in together}) == 3
    for prompt, sp, toks in zip(prompts, params, together):
        hist = []
        for step, tok in enumerate(toks):
            logits = pm.forward(cfg, W, prompt + toks[:step])[-1]
            logits = pm.apply_penalties(logits, hist[-sp.penalty_last_n:], sp.repetition_penalty, sp.frequency_penalty, sp.presence_penalty)
            w = pm.filtered_probs(logits, sp.temperature, sp.top_k, sp.top_p, sp.min_p)
            u = float(philox_uniform(np.array([sp.seed]), np.array([step]))[0])
            want = pm.cdf_walk(w, u)
            if tok != want:                                   # only a draw on the edge between two tokens may differ
                cum = torch.cumsum(w, 0) / w.sum()
                assert abs(tok - want) >= 1 and min(abs(float(cum[min(tok, want)]) - u), abs(float(cum[max(tok, want) - 1]) - u)) < 1e-4
                break
            hist.append(tok)


def test_stop_tokens_and_eos(model_folders, tmp_path):
    import shutil
    folder = str(tmp_path / "eos")
    shutil.copytree(model_folders["A"], folder)
    prompt = seeded_ids(90, 9, 512)
    free_run = plain_greedy(folder, prompt, 12)
    cfg = json.load(open(os.path.join(folder, "config.json")))
    cfg["eos_token_id"] = free_run[5]
    json.dump(cfg, open(os.path.join(folder, "config.json"), "w"))
    engine = Engine.load(folder, dtype="float32", kv_pages=16)
    first = free_run.index(free_run[5])
    out = engine.generate([prompt], SamplingParams(temperature=0.0, max_tokens=12))[0]
    assert out.finish_reason == "stop" and out.token_ids == free_run[: first + 1]
    out = engine.generate([prompt], SamplingParams(temperature=0.0, max_tokens=12, ignore_eos=True))[0]
    assert out.finish_reason == "length" and out.token_ids == free_run
    stop = free_run[2]
    out = engine.generate([prompt], SamplingParams(temperature=0.0, max_tokens=12, ignore_eos=True, stop_token_ids=(stop,)))[0]
    assert out.finish_reason == "stop" and out.token_ids == free_run[: free_run.index(stop) + 1]


def test_command_line(model_folders):
    folder = model_folders["A"]
    prompt = seeded_ids(95, 11, 512)
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "inferctl"), "completion", "--model", folder,
                           "--prompt-ids", ",".join(map(str, prompt)), "--max-tokens", "8", "--temperature", "0",
                           "--dtype", "float32", "--ignore-eos", "--stream", "--ctx-size", "256", "--max-parallel-sequences", "2"],
                          capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr
    lines = [json.loads(l) for l in proc.stdout.splitlines() if l.startswith("{")]
    want = plain_greedy(folder, prompt, 8)
    assert [l["token"] for l in lines if "token" in l] == want           # streamed one by one
    final = [l for l in lines if "token_ids" in l][0]
    assert final["token_ids"] == want and final["finish_reason"] == "length" and final["prompt_tokens"] == 11


def test_phase_timing_and_cache_planning(model_folders, capfd):
    folder = model_folders["C"]
    prompt = seeded_ids(97, 20, 777)
    plain = Engine.load(folder, dtype="float32", kv_pages=32, max_batch_size=2)
    want = plain.generate([prompt], SamplingParams(temperature=0.0, max_tokens=5, ignore_eos=True))[0].token_ids
    timed = Engine.load(folder, dtype="float32", max_batch_size=2, ctx_size=256, phase_timing=True)   # cache sized by the planner
    assert [p.num_pages for p in timed.runner.manager.pools] == [32, 32] and not timed.runner.decode_graphs
    got = timed.generate([prompt], SamplingParams(temperature=0.0, max_tokens=5, ignore_eos=True))[0].token_ids
    assert got == want
    assert timed.stats.steps == 5 and timed.stats.step_tokens == {32: 1, 1: 4}    # the prompt's 20 tokens, then one at a time
    err = capfd.readouterr().err
    assert "[phase_timing] #1 L=4 tokens=20" in err and "mixer=" in err and "lm_head=" in err
    t = timed.runner.timer
    assert t.forwards == 5 and all(t.totals[k] > 0 for k in ("embed", "norm", "mixer.qkv", "mixer.attention", "mixer", "ffn.gate_up",
                                                              "ffn", "final_norm", "lm_head"))
    assert abs(sum(t.shares().values()) - 1.0) < 1e-6


def test_logprobs_through_the_engine(model_folders):
    folder = model_folders["A"]
    cfg, W = pm.load_folder(folder, torch.float64)
    prompt = seeded_ids(98, 10, 512)
    engine = Engine.load(folder, dtype="float32", kv_pages=16)
    out = engine.generate([prompt], SamplingParams(temperature=0.0, max_tokens=6, ignore_eos=True, logprobs=3))[0]
    assert len(out.logprobs) == 6 and [l.token_id for l in out.logprobs] == out.token_ids
    for step, l in enumerate(out.logprobs):
        want = torch.log_softmax(pm.forward(cfg, W, prompt + out.token_ids[:step])[-1], -1)
        assert abs(l.logprob - float(want[l.token_id])) < 1e-4
        assert l.top_logprobs[0][0] == l.token_id and len(l.top_logprobs) == 3          # greedy: the sampled token is the top one
        assert all(abs(v - float(want[t])) < 1e-4 for t, v in l.top_logprobs)
    assert engine.generate([prompt], SamplingParams(temperature=0.0, max_tokens=2, ignore_eos=True))[0].logprobs is None


def _stateful_toy_runner(pages, slots, graph_safe=False, decode_graphs=True):
    """A two-layer model made outside the package: attention, then a mixer that keeps a decayed sum per request in a
    state slot (no cache).  A state that is not zero when a request starts changes every token after it.
    ``graph_safe``: the mixer takes steps of single tokens with device-side indexing only and says so, which lets
    the runner capture them."""
    from inferflux_amd.engine.model import Model
    from inferflux_amd.engine.runner import ModelRunner
    from inferflux_amd.parts import LayerSpec, Mixer, ModelPlan, ParamSpec, PartSpec, ScheduleEntry, StateSpec, register_part
    from inferflux_amd.parts.base import registered_parts

    H, V, kind = 32, 61, "toy_decay_sum_for_generation" + ("_in_graphs" if graph_safe else "")
    if kind not in registered_parts("mixer"):
        from inferflux_amd.kernels import ops

        @register_part("mixer", kind)
        class DecaySum(Mixer):
            def __init__(self, name, hidden_size, decay):
                self.name, self.H, self.decay = name, hidden_size, decay
                self.graph_safe = graph_safe
            def param_specs(self):
                return {f"{self.name}.mix.weight": ParamSpec((self.H, self.H), ("normal", 0.3))}
            def load(self, tensors):
                self.w = tensors[f"{self.name}.mix.weight"]
            def state_spec(self):
                return StateSpec((self.H,), "float32")
            def forward(self, h, ctx, binding):
                if self.graph_safe and ctx.n_tokens == ctx.n_requests:
                    # one token each: the slots come from the step's device array, so a replayed graph follows them
                    slots = ctx.state_slots.long()
                    s = binding.state.index_select(0, slots) * self.decay + h.float()
                    binding.state.index_copy_(0, slots, s)
                    return ops.gemm_f32(s.to(h.dtype), self.w)
                out = torch.empty_like(h)
                for r in range(ctx.n_requests):
                    s = binding.state[int(ctx.h_state_slots[r])]
                    a, n = int(ctx.h_q_start[r]), int(ctx.h_q_len[r])
                    for t in range(a, a + n):
                        s.mul_(self.decay).add_(h[t].float())
                        out[t] = s.to(h.dtype)
                return out @ self.w.t()

    def layer(i, mixer):
        p = f"toy.layers.{i}"
        return LayerSpec(p, PartSpec("prenorm"), PartSpec("rmsnorm", {"name": f"{p}.n1", "eps": 1e-5}), mixer,
                         PartSpec("rmsnorm", {"name": f"{p}.n2", "eps": 1e-5}),
                         PartSpec("swiglu", {"name": f"{p}.mlp", "intermediate_size": 48}))

    attn = PartSpec("paged_attention", {"name": "toy.layers.0.attn", "n_heads": 2, "n_kv_heads": 1, "head_dim": 16,
                                        "bias": False, "position": PartSpec("rotary", {"head_dim": 16, "theta": 100.0})})
    plan = ModelPlan(vocab_size=V, hidden_size=H, max_position=256,
                     embedding=PartSpec("token_embedding", {"name": "toy.embed", "vocab_size": V}),
                     layers=(layer(0, attn), layer(1, PartSpec(kind, {"name": "toy.layers.1.mixer", "decay": 0.95}))),
                     schedule=(ScheduleEntry(0), ScheduleEntry(1)),
                     final_norm=PartSpec("rmsnorm", {"name": "toy.norm", "eps": 1e-5}),
                     lm_head=PartSpec("linear_head", {"name": "toy.head", "vocab_size": V}))
    model = Model(plan=plan).init_random(4, torch.float32, "cuda")
    return ModelRunner(model, num_pages=pages, max_requests=slots, decode_graphs=decode_graphs), V


def test_a_model_with_state_keeps_padded_decode_graphs():
    """Six requests with limits of their own, so that the batch shrinks from 6 to 1: the captured steps' batches are
    filled up to 8, 4, 2 and 1 with rows that use a state slot no request holds, so four layouts serve every size;
    tokens are those of eager steps, and nothing is started early (a step over state cannot be run twice)."""
    from inferflux_amd.engine.engine import Engine as Eng
    from inferflux_amd.engine.scheduler import SchedulerConfig
    lens, limits = [12, 30, 7, 21, 16, 9], [40, 33, 26, 19, 12, 6]

    def run(**kw):
        runner, V = _stateful_toy_runner(pages=64, slots=6, graph_safe=True, **kw)
        eng = Eng(runner, SchedulerConfig(6, 4096, 512))
        params = [SamplingParams(temperature=0.0, max_tokens=n, ignore_eos=True) for n in limits]
        outs = eng.generate([seeded_ids(700 + i, n, V) for i, n in enumerate(lens)], params)
        runner.manager.check()
        assert runner.manager.free_pages() == [64]
        return [o.token_ids for o in outs], runner

    want, eager = run(decode_graphs=False)
    assert eager.graph_captures == 0 and [len(t) for t in want] == limits
    got, runner = run()
    assert runner.model.graph_safe and runner.storage.has_state and not runner.starts_steps_early
    assert got == want
    assert 1 <= runner.graph_captures <= 4 and runner.graph_replays >= 30
    # the rows that stand for nobody wrote to the slot beyond the requests' and to no other
    state = next(iter(runner.storage._states.values()))
    assert state.shape[0] == 7 and float(state[6].abs().max()) > 0


def test_per_request_state_is_zero_for_every_admission_through_the_engine():
    """Requests admitted by the scheduler (not through the runner's add_request): into a slot another request has
    left, and again after a preemption.  Each one's tokens must be those of the same request alone in a fresh engine."""
    from inferflux_amd.engine.engine import Engine as Eng
    from inferflux_amd.engine.scheduler import SchedulerConfig
    lens, n_new = [30, 9, 40, 22, 35], 24
    sp = SamplingParams(temperature=0.0, max_tokens=n_new, ignore_eos=True)
    want = []
    for i, n in enumerate(lens):
        runner, V = _stateful_toy_runner(pages=16, slots=1)
        want.append(Eng(runner, SchedulerConfig(1, 4096, 512)).generate([seeded_ids(500 + i, n, V)], sp)[0].token_ids)
    assert len({tuple(w) for w in want}) == len(want)
    prompts = [seeded_ids(500 + i, n, V) for i, n in enumerate(lens)]
    # two slots for five requests: three of them start in a slot that holds another request's last state
    runner, _ = _stateful_toy_runner(pages=32, slots=2)
    eng = Eng(runner, SchedulerConfig(2, 4096, 16, 16))
    assert not runner.starts_steps_early                      # a step over state cannot be run twice
    outs = eng.generate(prompts, sp)
    assert [o.token_ids for o in outs] == want and eng.stats.preemptions == 0
    # three slots and 7 pages: 30+24, 9+24 and 40+24 tokens need 4 + 3 + 4 pages, so somebody is preempted and
    # admitted again (its slot may be the one it had: the state it left there must not survive)
    runner, _ = _stateful_toy_runner(pages=7, slots=3)
    eng = Eng(runner, SchedulerConfig(3, 4096, 16, 16))
    outs = eng.generate(prompts, sp)
    assert eng.stats.preemptions >= 1 and any(o.preemptions for o in outs)
    assert [o.token_ids for o in outs] == want
    runner.manager.check()
    assert runner.manager.free_pages() == [7]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("early", [True, False])
def test_requests_added_and_aborted_between_steps_by_hand(early, dtype, model_folders):
    """The engine driven step by step: a request arrives between two decode steps (the step that was started early
    for the others is void), a running request is aborted right after a step that started the next one early (its
    row of that step is dropped), a waiting one is aborted before it ever ran, greedy requests run beside a seeded
    one.  Survivors' tokens are the plain model's; aborted requests return what they had.  In bfloat16 (configuration A,
    whose head size the matrix-core kernels take) every token is within rounding of the plain model's best for the
    prefix it follows."""
    name = "B" if dtype == "float32" else "A"
    folder, V = model_folders[name], TINY[name]["vocab_size"]
    cfg, W = pm.load_folder(folder, torch.float64)
    P = {k: seeded_ids(600 + i, n, V) for i, (k, n) in enumerate({"a": 21, "b": 5, "c": 33, "d": 12, "w": 8, "s": 17, "x": 9}.items())}
    greedy = lambda n: SamplingParams(temperature=0.0, max_tokens=n, ignore_eos=True)
    eng = Engine.load(folder, dtype=dtype, kv_pages=40, max_batch_size=4, chunked_prefill_tokens=16, prefill_tokens_alone=16,
                      start_steps_early=early)
    runner = eng.runner
    done = {}

    def right(rid, tokens, n):
        if dtype == "bfloat16":
            return near_best(cfg, W, P[rid], tokens, name)
        return tokens == plain_greedy(folder, P[rid], n)[:len(tokens)]

    def step(n=1):
        for _ in range(n):
            for o in eng.step():
                done[o.request_id] = o

    eng.add_request(P["a"], greedy(30), "a")
    eng.add_request(P["b"], greedy(30), "b")
    eng.add_request(P["s"], SamplingParams(temperature=0.9, top_p=0.95, seed=77, max_tokens=12, ignore_eos=True), "s")
    step(6)                                                    # prompts are in, everyone decodes
    if early:
        assert runner._launched is not None                    # the next step of a, b, s is already running
    eng.add_request(P["c"], greedy(10), "c")                   # an arrival: that step is void
    step(1)
    assert runner.has_request("c")
    step(5)
    if early:
        assert runner._launched is not None and "b" in runner._launched[0][0]
    out_b = eng.abort("b")                                     # b's row of the step that is running is dropped
    assert out_b.finish_reason == "abort" and not runner.has_request("b") and len(out_b.token_ids) >= 5
    step(2)
    # s has reached its limit; d and w fill the batch (a, c, d, w), x waits and is aborted before it ever ran
    assert "s" in done and len(eng.scheduler.running) == 2
    eng.add_request(P["d"], greedy(8), "d")
    eng.add_request(P["w"], greedy(8), "w")
    eng.add_request(P["x"], greedy(8), "x")
    step(1)
    assert runner.has_request("d") and runner.has_request("w") and not runner.has_request("x") and len(eng.scheduler.waiting) == 1
    out_x = eng.abort("x")
    assert out_x.finish_reason == "abort" and out_x.token_ids == [] and not eng.scheduler.waiting
    assert eng.abort("x") is None and eng.abort("nobody") is None
    while eng.has_unfinished():
        step(1)
    runner.manager.check()
    assert runner.manager.free_pages() == [40] and not runner.manager.live()
    for k, n in (("a", 30), ("c", 10), ("d", 8), ("w", 8)):
        assert done[k].finish_reason == "length" and len(done[k].token_ids) == n and right(k, done[k].token_ids, n), k
    assert right("b", out_b.token_ids, 30)
    if dtype == "float32":
        # the seeded request alone gives the same tokens: neither the batch nor the arrivals and aborts around it matter
        alone = Engine.load(folder, dtype="float32", kv_pages=40, max_batch_size=4)
        assert alone.generate([P["s"]], SamplingParams(temperature=0.9, top_p=0.95, seed=77, max_tokens=12, ignore_eos=True))[0].token_ids \
            == done["s"].token_ids


def near_best(cfg, W, prompt, tokens, name):
    """Whether every token of ``tokens`` is, for the prefix before it, within rounding of the plain model's best
    token: its logit at most twice the bfloat16 bound of the configuration below the largest one.  (Among the
    hundreds of a tiny vocabulary one to three tokens are; the logits of a wrong prefix, page or position put their
    own best there with a chance of well under a hundredth.)"""
    from conftest import tol
    if not tokens:
        return True
    full = pm.forward(cfg, W, list(prompt) + list(tokens))
    for i, tok in enumerate(tokens):
        row = full[len(prompt) - 1 + i]
        if row[tok] < row.max() - 2 * tol("bfloat16", name) * row.abs().max():
            return False
    return True


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("early", [True, False], ids=["early", "late"])
@pytest.mark.parametrize("name,seed", [("C", 2), ("A", 3)])
def test_random_arrivals_aborts_priorities_and_preemptions(name, seed, early, dtype, model_folders):
    """Forty requests of random lengths, limits and priorities arrive at random steps and some are aborted at random,
    through a cache too small for them (requests are preempted and recomputed).  In float32 every finished request's
    tokens are the plain model's and every aborted one's a beginning of them; in bfloat16 (the matrix-core kernels,
    decode steps as replayed graphs with their batches filled up, steps started early and made void) every token is
    within rounding of the plain model's best for the prefix it follows.  The cache's books are right after every
    step and every pool is whole at the end."""
    import random
    folder, V = model_folders[name], TINY[name]["vocab_size"]
    cfg, W = pm.load_folder(folder, torch.float64)
    rng = random.Random(seed * 7 + (1 if early else 0))
    pages = rng.randint(14, 22)
    batch, chunk = rng.randint(3, 6), rng.choice([8, 16, 24, 48])
    eng = Engine.load(folder, dtype=dtype, kv_pages=pages, max_batch_size=batch,
                      chunked_prefill_tokens=chunk, max_batch_tokens=rng.choice([32, 64, 256]),
                      prefill_tokens_alone=3 * chunk, start_steps_early=early)
    reqs, done, aborted = {}, {}, {}
    n_req, next_id, steps = 40, 0, 0
    while next_id < n_req or eng.has_unfinished():
        steps += 1
        for _ in range(rng.choice([0, 0, 0, 1, 1, 2, 3])):
            if next_id < n_req:
                n_new = rng.randint(1, 30)
                prompt = seeded_ids(seed * 1000 + next_id, rng.randint(1, min(110, pages * 16 - n_new - 1)), V)
                eng.add_request(prompt, SamplingParams(temperature=0.0, max_tokens=n_new, ignore_eos=True), f"r{next_id}",
                                priority=rng.choice([0, 0, 0, 1, 2]))
                reqs[f"r{next_id}"] = (prompt, n_new)
                next_id += 1
        live = [r for r in reqs if r not in done and r not in aborted]
        if live and rng.random() < 0.08:
            rid = rng.choice(live)
            out = eng.abort(rid)
            if out is not None:
                aborted[rid] = out
        for o in eng.step():
            done[o.request_id] = o
        eng.runner.manager.check()
        assert steps < 5000, "the engine makes no progress"
    assert eng.runner.manager.free_pages() == [pages] * len(eng.runner.manager.groups) and not eng.runner.manager.live()
    assert set(done) | set(aborted) == set(reqs) and not set(done) & set(aborted)
    assert eng.stats.preemptions > 0 and aborted and len(done) > 10          # the run did meet what it is about
    if dtype == "bfloat16":
        assert eng.runner.decode_graphs and eng.runner.graph_replays > 20
    for rid, (prompt, n_new) in reqs.items():
        out = done.get(rid) or aborted[rid]
        assert out.finish_reason == ("length" if rid in done else "abort") and len(out.token_ids) <= n_new
        assert rid in aborted or len(out.token_ids) == n_new
        if dtype == "bfloat16":
            assert near_best(cfg, W, prompt, out.token_ids, name), (rid, out.token_ids)
            continue
        want = pm.greedy_generate(cfg, W, prompt, n_new)
        assert out.token_ids == want[:len(out.token_ids)], rid


def test_a_seeded_request_with_penalties_keeps_its_tokens_across_a_preemption(model_folders):
    """A request that samples (temperature 0.9, a seed, a repetition penalty and a frequency penalty) is preempted and
    recomputed in a pool too small for the three that run: its draw counter and the history its penalties read
    outlive the preemption, so its tokens are those of the same request in a roomy pool (float32: the logits of a
    position are the same bits however it was reached).  The invariant of the reference's sampler test, extended
    over a preemption (tests/unit/test_gpu_sampler.cpp:205-262)."""
    folder, V = model_folders["A"], TINY["A"]["vocab_size"]
    prompts = [seeded_ids(820 + i, 40, V) for i in range(3)]

    def params():
        return [SamplingParams(temperature=0.0, max_tokens=40, ignore_eos=True),
                SamplingParams(temperature=0.0, max_tokens=40, ignore_eos=True),
                SamplingParams(temperature=0.9, seed=4711, repetition_penalty=1.3, frequency_penalty=0.2, penalty_last_n=16,
                               max_tokens=40, ignore_eos=True)]

    def run(pages):
        eng = Engine.load(folder, dtype="float32", kv_pages=pages, max_batch_size=4)
        ids = [eng.add_request(p, sp, priority=pr) for p, sp, pr in zip(prompts, params(), (1, 1, 0))]   # the sampler goes first
        outs = {}
        while eng.has_unfinished():
            for o in eng.step():
                outs[o.request_id] = o
        eng.runner.manager.check()
        assert eng.runner.manager.free_pages() == [pages]
        return [outs[i] for i in ids]

    roomy, tight = run(64), run(8)                             # 15 pages would be needed
    assert roomy[2].preemptions == 0 and tight[2].preemptions >= 1
    assert [o.token_ids for o in tight] == [o.token_ids for o in roomy]
    alone = Engine.load(folder, dtype="float32", kv_pages=64, max_batch_size=4).generate([prompts[2]], [params()[2]])[0]
    assert alone.token_ids == roomy[2].token_ids and len(set(alone.token_ids)) > 8
