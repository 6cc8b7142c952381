"""The engine in one process: the step function against the plain model, each part alone, long
decoding, the first tokens, and a toy mixer with state of its own built from outside the package."""
import math

import pytest
import torch

import plain_model as pm
from conftest import REL_TOL, TINY, plain_logits, rel_err, seeded_ids, tol

pytestmark = pytest.mark.gpu

if torch.cuda.is_available():
    from inferflux_amd.cache import OutOfPages
    from inferflux_amd.engine.api import load_runner
    from inferflux_amd.engine.context import StepEntry
    from inferflux_amd.engine.runner import StepError

DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def run_whole(runner, rid, ids):
    runner.add_request(rid)
    out = runner.step([StepEntry(rid, ids, list(range(len(ids))))]).cpu()
    runner.free_request(rid)
    return out


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(TINY))
def test_whole_prompt(name, dtype, sharp_folders):
    folder = sharp_folders[name, dtype]
    runner = load_runner(folder, DT[dtype], num_pages=32)
    for n in (1, 2, 29, 200):
        ids = seeded_ids(n, n, TINY[name]["vocab_size"])
        got = run_whole(runner, "a", ids)
        assert rel_err(got, plain_logits(folder, ids)) < tol(dtype, name), (name, n)
    runner.manager.check()
    assert runner.manager.free_pages() == [32] * len(runner.manager.groups)


@pytest.mark.parametrize("name", list(TINY))
def test_first_tokens_and_single_token_prompt(name, sharp_folders):
    """Position 0 has one key (itself); its logits depend on the token alone."""
    folder = sharp_folders[name]
    runner = load_runner(folder, torch.float32, num_pages=8)
    for tok in (0, 7, TINY[name]["vocab_size"] - 1):
        a = run_whole(runner, "x", [tok])
        b = run_whole(runner, "y", [tok, 3, 4])
        assert rel_err(a, plain_logits(folder, [tok])) < REL_TOL["float32"]
        assert torch.equal(a[0], b[0])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_stays_on_the_plain_model(dtype, sharp_folders):
    folder, name = sharp_folders["C", dtype], "C"
    runner = load_runner(folder, DT[dtype], num_pages=24)
    ids = seeded_ids(11, 300, TINY[name]["vocab_size"])
    want = plain_logits(folder, ids)
    runner.add_request("d")
    got = [runner.step([StepEntry("d", ids[:5], [4])]).cpu()[0]]
    for p in range(5, 300):
        got.append(runner.step([StepEntry("d", [ids[p]], [0])]).cpu()[0])
        runner.manager.check()
    assert rel_err(torch.stack(got), want[4:]) < tol(dtype, name)
    # the windowed group kept only the pages a window of 24 can still see
    held = sum(1 for p in runner.manager.block_table("d", 1) if p >= 0)
    assert held <= 24 // 16 + 2 and sum(1 for p in runner.manager.block_table("d", 0) if p >= 0) == -(-300 // 16)


def test_float32_results_do_not_depend_on_the_cutting_bit_for_bit(sharp_folders):
    folder = sharp_folders["A"]
    runner = load_runner(folder, torch.float32, num_pages=32)
    ids = seeded_ids(12, 150, 512)
    whole = run_whole(runner, "w", ids)
    runner.add_request("filler")                           # other pages, another batch composition
    runner.step([StepEntry("filler", ids[:37], [])])
    runner.add_request("c")
    rows, p = [], 0
    for m in (64, 1, 2, 17, 1, 65):
        rows.append(runner.step([StepEntry("filler", [5], [0]), StepEntry("c", ids[p:p + m], list(range(m)))]).cpu()[1:])
        p += m
    assert torch.equal(torch.cat(rows), whole)


def test_step_refuses_bad_input_and_changes_nothing(sharp_folders):
    runner = load_runner(sharp_folders["A"], torch.float32, num_pages=4)
    runner.add_request("a")
    with pytest.raises(StepError, match="outside"):
        runner.step([StepEntry("a", [1, 512], [0])])
    with pytest.raises(StepError, match="not live"):
        runner.step([StepEntry("b", [1], [0])])
    with pytest.raises(StepError, match="wanted places"):
        runner.step([StepEntry("a", [1, 2], [2])])
    with pytest.raises(StepError, match="twice"):
        runner.step([StepEntry("a", [1], []), StepEntry("a", [2], [])])
    with pytest.raises(StepError, match="max_position"):
        runner.step([StepEntry("a", [1] * 257, [])])
    with pytest.raises(OutOfPages):
        runner.step([StepEntry("a", [1] * 65, [])])       # 5 pages wanted, 4 in the pool
    assert runner.length("a") == 0 and runner.manager.free_pages() == [4]
    runner.step([StepEntry("a", [1] * 64, [63])])
    assert runner.manager.free_pages() == [0]
    runner.manager.check()


# ---- parts alone ----------------------------------------------------------------------------
def test_parts_alone(sharp_folders):
    """Each part of a layer against its plain function, on the layer's own weights."""
    from inferflux_amd.engine.context import StepContext
    folder = sharp_folders["B"]
    cfg, W = pm.load_folder(folder, torch.float64)
    runner = load_runner(folder, torch.float32, num_pages=16)
    model = runner.model
    ids = seeded_ids(13, 40, 1000)
    runner.add_request("p")
    runner.manager.reserve("p", len(ids))
    ctx = StepContext([StepEntry("p", ids, [0, 39])], runner.manager, torch.float32, runner.device)
    dev = runner.device
    g = torch.Generator().manual_seed(14)
    x = torch.randn(40, 144, generator=g)
    blk, p = model.blocks[1], "model.layers.1"
    # embedding
    assert torch.equal(model.embedding.forward(ctx).cpu().double(), W["model.embed_tokens.weight"][ids])
    # norm (with and without a pending delta)
    delta = torch.randn(40, 144, generator=g)
    res = x.to(dev).clone()
    got = blk.norm_in.forward(res, delta.to(dev), torch.float32).cpu().double()
    assert torch.allclose(got, pm.rms_norm((x + delta).double(), W[f"{p}.input_layernorm.weight"], cfg["rms_norm_eps"]), atol=1e-5)
    # feed-forward
    got = blk.ffn.forward(x.to(dev), ctx).cpu().double()
    want = pm.swiglu(x.double(), W[f"{p}.mlp.gate_proj.weight"], W[f"{p}.mlp.up_proj.weight"], W[f"{p}.mlp.down_proj.weight"])
    assert torch.allclose(got, want, rtol=1e-4, atol=1e-5)
    # mixer (attention with bias, rotary and cache write) on arbitrary input rows
    got = blk.mixer.forward(x.to(dev), ctx, runner.storage.binding(1)).cpu().double()
    want = pm.attention_block(x.double(), W, cfg, 1, list(range(40)))
    assert torch.allclose(got, want, rtol=1e-4, atol=1e-5)
    # head
    h = torch.randn(3, 144, generator=g)
    assert torch.allclose(model.head.forward(h.to(dev)).cpu().double(), h.double() @ W["lm_head.weight"].t(), rtol=1e-4, atol=1e-5)


# ---- a toy mixer with state of its own --------------------------------------------------------
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_toy_mixer_with_state_registers_builds_and_steps(tmp_path, dtype):
    """A mixer defined here (a running decayed sum per request, kept in a state slot, no cache) is
    registered, put into a plan beside an attention layer, built, loaded and stepped, without any
    change to the package.  Its result must not depend on how the sequence is cut.  In bfloat16 the
    package's own parts hand each other rows whose norm is still to be finished when a step is short;
    the toy mixer, which declares nothing of that, is given finished rows in the same model."""
    from inferflux_amd.config.base import ModelConfig
    from inferflux_amd.engine.model import Model
    from inferflux_amd.engine.runner import ModelRunner
    from inferflux_amd.parts import (LayerSpec, Mixer, ModelPlan, ParamSpec, PartSpec, ScheduleEntry, StateSpec,
                                     register_part)

    H, V = 32, 50

    kind = f"toy_decay_sum_{dtype}"

    @register_part("mixer", kind)
    class DecaySum(Mixer):
        def __init__(self, name, hidden_size, decay):
            self.name, self.H, self.decay = name, hidden_size, decay
        def param_specs(self):
            return {f"{self.name}.mix.weight": ParamSpec((self.H, self.H))}
        def load(self, tensors):
            self.w = tensors[f"{self.name}.mix.weight"]
        def state_spec(self):
            return StateSpec((self.H,), "float32")
        def forward(self, h, ctx, binding):
            out = torch.empty_like(h)
            for r in range(ctx.n_requests):                       # rows of a request in position order
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
    plan = ModelPlan(vocab_size=V, hidden_size=H, max_position=128,
                     embedding=PartSpec("token_embedding", {"name": "toy.embed", "vocab_size": V}),
                     layers=(layer(0, attn), layer(1, PartSpec(kind, {"name": "toy.layers.1.mixer", "decay": 0.9}))),
                     schedule=(ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(0, cache_from=0), ScheduleEntry(1)),
                     final_norm=PartSpec("rmsnorm", {"name": "toy.norm", "eps": 1e-5}),
                     lm_head=PartSpec("linear_head", {"name": "toy.head", "vocab_size": V}))
    model = Model(plan=plan).init_random(3, DT[dtype], "cuda")
    runner = ModelRunner(model, num_pages=16, max_requests=3)
    assert [g.entries for g in runner.storage.groups] == [(0,)]          # one cache owner; entry 2 reads it
    assert runner.storage.binding(2).writes_cache is False and runner.storage.binding(2).cache is runner.storage.binding(0).cache
    assert runner.storage.binding(1).state.shape == (3 + 1, H)           # (one slot more: for the rows that stand for nobody)
    assert runner.storage.binding(3).state is not runner.storage.binding(1).state
    ids = seeded_ids(15, 60, V)
    runner.add_request("w")
    whole = runner.step([StepEntry("w", ids, list(range(60)))]).cpu()
    runner.free_request("w")
    runner.add_request("other"); runner.add_request("c")                 # "c" reuses the slot "w" left: state must be zero
    rows, p = [], 0
    for m in (7, 1, 2, 30, 1, 19):
        out = runner.step([StepEntry("other", ids[p:p + 1], []), StepEntry("c", ids[p:p + m], list(range(m)))])
        rows.append(out.cpu()); p += m
    if dtype == "float32":
        assert torch.allclose(torch.cat(rows), whole, rtol=1e-4, atol=1e-5)
    else:
        assert rel_err(torch.cat(rows), whole) < REL_TOL["bfloat16"]
    assert not torch.allclose(whole[1:], whole[:-1])


def test_a_layer_that_reads_another_entries_cache_in_bfloat16():
    """The schedule runs one attention layer twice, the second time on the first one's cache (queries only).  In
    bfloat16 with a head size of 32, steps of up to 16 tokens take the fused projection + rotation kernel and longer
    ones the separate kernels: both must give the same logits within bfloat16's rounding."""
    from inferflux_amd.engine.model import Model
    from inferflux_amd.engine.runner import ModelRunner
    from inferflux_amd.parts import LayerSpec, ModelPlan, PartSpec, ScheduleEntry

    H, V = 64, 90
    p = "twice.layers.0"
    attn = PartSpec("paged_attention", {"name": f"{p}.attn", "n_heads": 4, "n_kv_heads": 2, "head_dim": 32, "bias": True,
                                        "position": PartSpec("rotary", {"head_dim": 32, "theta": 1000.0})})
    layer = LayerSpec(p, PartSpec("prenorm"), PartSpec("rmsnorm", {"name": f"{p}.n1", "eps": 1e-5}), attn,
                      PartSpec("rmsnorm", {"name": f"{p}.n2", "eps": 1e-5}),
                      PartSpec("swiglu", {"name": f"{p}.mlp", "intermediate_size": 80}))
    plan = ModelPlan(vocab_size=V, hidden_size=H, max_position=128,
                     embedding=PartSpec("token_embedding", {"name": "twice.embed", "vocab_size": V}),
                     layers=(layer,), schedule=(ScheduleEntry(0), ScheduleEntry(0, cache_from=0)),
                     final_norm=PartSpec("rmsnorm", {"name": "twice.norm", "eps": 1e-5}),
                     lm_head=PartSpec("linear_head", {"name": "twice.head", "vocab_size": V}))
    logits = {}
    for dtype in (torch.float32, torch.bfloat16):
        model = Model(plan=plan).init_random(5, dtype, "cuda")
        runner = ModelRunner(model, num_pages=16, max_requests=2)
        ids = seeded_ids(21, 56, V)
        runner.add_request("w")
        whole = runner.step([StepEntry("w", ids, list(range(56)))]).cpu()
        runner.free_request("w")
        runner.add_request("c")
        rows, at = [], 0
        for m in (1, 2, 16, 5, 16, 16):
            rows.append(runner.step([StepEntry("c", ids[at:at + m], list(range(m)))]).cpu()); at += m
        logits[dtype] = (whole, torch.cat(rows))
    w32, c32 = logits[torch.float32]
    wb, cb = logits[torch.bfloat16]
    assert torch.equal(w32, c32)
    assert rel_err(cb, w32) < REL_TOL["bfloat16"] and rel_err(wb, w32) < REL_TOL["bfloat16"]


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_steps_of_few_rows_need_no_kernel_for_the_norms_between_products(name, sharp_folders, monkeypatch):
    """In bfloat16 a step of up to 16 rows adds each sub-block's output to the stream in its last product's epilogue
    and applies the next norm's factor in the next product; the embedding prepares the first layer's first norm the
    same way and the head takes the final norm's rows (these steps want every row's logits): no norm keeps a kernel.
    Logits agree with the plain model, and with the same step run with a kernel for every norm."""
    from inferflux_amd.kernels import ops
    folder, V, L = sharp_folders[name, "bfloat16"], TINY[name]["vocab_size"], TINY[name]["num_hidden_layers"]
    ids = seeded_ids(31, 60, V)
    want = plain_logits(folder, ids)
    calls = []
    real = ops.add_rmsnorm
    monkeypatch.setattr(ops, "add_rmsnorm", lambda *a, **k: (calls.append(a[0].shape[0]), real(*a, **k))[1])

    def run(runner):
        runner.decode_graphs = False              # every step eagerly: replays call nothing from Python
        runner.add_request("n")
        out, at = [], 0
        for m in (17, 16, 1, 9, 16, 1):
            calls.clear()
            out.append(runner.step([StepEntry("n", ids[at:at + m], list(range(m)))]).cpu()); at += m
            yield_calls.append((m, len(calls)))
        runner.free_request("n")
        return torch.cat(out)

    yield_calls = []
    fused = run(load_runner(folder, torch.bfloat16, num_pages=16))
    assert yield_calls == [(17, 2 * L + 1)] + [(m, 0) for m in (16, 1, 9, 16, 1)], yield_calls
    monkeypatch.setattr(ops, "adds_into_stream", lambda *a: False)
    monkeypatch.setattr(ops, "takes_scaled_rows", lambda *a: False)
    yield_calls = []
    separate = run(load_runner(folder, torch.bfloat16, num_pages=16))
    assert all(n == 2 * L + 1 for _, n in yield_calls), yield_calls
    assert rel_err(fused, want[:60]) < tol("bfloat16", name) and rel_err(separate, want[:60]) < tol("bfloat16", name)
    assert rel_err(fused, separate) < tol("bfloat16", name)


def test_a_decode_step_started_before_the_host_has_its_tokens(sharp_folders):
    """launch_prepared starts the prepared step with tokens that are on the GPU only; step hands out its logits for
    the same requests, or the rows of those that are left of them, and computes anything else afresh: bit for bit
    the logits of steps that were not started early."""
    folder, V = sharp_folders["C", "float32"], TINY["C"]["vocab_size"]
    ids = {r: seeded_ids(40 + i, 70, V) for i, r in enumerate("abc")}
    order = ["abc", "abc", "abc", "acb", "ab", "ab", "ab", "abc", "abc", "c"]

    def run(early):
        runner = load_runner(folder, torch.float32, num_pages=24)
        out, outcome = [], []
        for r in "abc":
            runner.add_request(r)
            runner.step([StepEntry(r, ids[r][:30], [])])
        at = {r: 30 for r in "abc"}
        for k, who in enumerate(order):
            started = False
            if early and k > 0:
                guess = order[k - 1]
                assert runner.prepare_decode(list(guess)) is True
                tokens = torch.tensor([ids[r][at[r]] for r in guess], dtype=torch.int32, device="cuda")
                started = runner.launch_prepared(tokens)
                assert (runner._launched is not None) == started and (runner._prepared is None) == started
            got = []
            real = runner._take_launched
            runner._take_launched = lambda e: (got.append(real(e)), got[0])[1]
            out.append(runner.step([StepEntry(r, [ids[r][at[r]]], [0]) for r in who]).cpu())
            del runner._take_launched
            assert len(got) == int(started)
            outcome.append("-" if not started else "void" if got[0] is None else "taken")
            assert runner._launched is None and runner._prepared is None
            for r in who:
                at[r] += 1
            runner.manager.check()
        for r in "abc":
            runner.free_request(r)
        runner.manager.check()
        assert runner.manager.free_pages() == [24] * len(runner.manager.groups)
        return out, outcome

    plain, _ = run(False)
    early, outcome = run(True)
    #          abc  abc      abc      acb (order)  ab of acb  ab (no graph yet)  ab   abc of ab  abc      c of abc
    assert outcome == ["-", "taken", "taken", "void", "taken", "-", "taken", "void", "taken", "taken"]
    for a, b in zip(plain, early):
        assert torch.equal(a, b)
    # tokens of another kind or number are refused, and so is a model whose mixers keep state of their own
    runner = load_runner(folder, torch.float32, num_pages=24)
    runner.add_request("x")
    runner.step([StepEntry("x", ids["a"][:30], [])])
    runner.step([StepEntry("x", [ids["a"][30]], [0])])                     # captures the graph of this layout
    assert runner.prepare_decode(["x"])
    assert not runner.launch_prepared(torch.zeros(2, dtype=torch.int32, device="cuda"))
    assert not runner.launch_prepared(torch.zeros(1, dtype=torch.int64, device="cuda"))
    assert not runner.launch_prepared(torch.zeros(1, dtype=torch.int32))
    # a step that brings other tokens than the early one ran on is computed afresh, with its own tokens
    started_on = torch.tensor([ids["a"][31]], dtype=torch.int32, device="cuda")
    assert runner.launch_prepared(started_on)
    other = (ids["a"][31] + 1) % V
    got = runner.step([StepEntry("x", [other], [0])]).cpu()
    fresh = load_runner(folder, torch.float32, num_pages=24)
    fresh.add_request("y")
    fresh.step([StepEntry("y", ids["a"][:31], [])])
    assert torch.equal(got, fresh.step([StepEntry("y", [other], [0])]).cpu())
    assert runner.length("x") == 32
    assert runner.prepare_decode(["x"])
    runner.storage._states[0] = torch.zeros(1, device="cuda")
    assert not runner.launch_prepared(torch.zeros(1, dtype=torch.int32, device="cuda")) and runner._prepared is not None


def test_a_decode_step_got_ready_ahead_of_its_tokens(sharp_folders):
    """prepare_decode does, before the tokens are known, what a step of single tokens needs besides them; step uses
    it for exactly that step and falls back to the ordinary path for any other, with the same logits either way."""
    folder, V = sharp_folders["C", "float32"], TINY["C"]["vocab_size"]
    ids = {r: seeded_ids(40 + i, 70, V) for i, r in enumerate("abc")}

    def run(prepare):
        runner = load_runner(folder, torch.float32, num_pages=24)
        out, used = [], 0
        for r in "abc":
            runner.add_request(r)
            runner.step([StepEntry(r, ids[r][:30], [])])
        order = ["abc", "abc", "abc", "acb", "ab", "ab", "abc", "abc"]       # same step, same, same, other order, fewer, ...
        at = {r: 30 for r in "abc"}
        for k, who in enumerate(order):
            if prepare and k > 0:
                assert runner.prepare_decode(list(order[k - 1])) is True    # the guess: the last step's requests again
            entries = [StepEntry(r, [ids[r][at[r]]], [0]) for r in who]
            was = runner._prepared is not None
            out.append(runner.step(entries).cpu())
            used += int(was and who == order[k - 1])
            assert runner._prepared is None
            for r in who:
                at[r] += 1
            runner.manager.check()
        if prepare:                                                        # got ready for "b" alone, given two tokens of "b"
            runner.prepare_decode(["b"])
            out.append(runner.step([StepEntry("b", ids["b"][at["b"]:at["b"] + 2], [0, 1])]).cpu())
        else:
            out.append(runner.step([StepEntry("b", ids["b"][at["b"]:at["b"] + 2], [0, 1])]).cpu())
        for r in "abc":
            runner.free_request(r)
        runner.manager.check()
        assert runner.manager.free_pages() == [24] * len(runner.manager.groups)
        return out, used

    plain, _ = run(False)
    ahead, used = run(True)
    assert used == 4
    for a, b in zip(plain, ahead):
        assert torch.equal(a, b)
    want = plain_logits(folder, ids["a"][:38])
    assert rel_err(torch.stack([o[0] for o in plain[:8]]), want[30:38]) < REL_TOL["float32"]
    # what it cannot get ready it leaves alone: a request that is not live, one named twice, no pages left
    runner = load_runner(folder, torch.float32, num_pages=2)
    runner.add_request("x")
    runner.step([StepEntry("x", ids["a"][:32], [])])                       # both pages of both groups are full
    free = runner.manager.free_pages()
    assert runner.prepare_decode(["x"]) is False and runner.prepare_decode(["x", "x"]) is False
    assert runner.prepare_decode(["nobody"]) is False and runner.manager.free_pages() == free
    with pytest.raises(OutOfPages):
        runner.step([StepEntry("x", [5], [0])])


@pytest.mark.parametrize("copy", [True, False])
@pytest.mark.parametrize("name", ["B", "C"])
def test_portions_of_every_product_size_with_and_without_the_decode_copy(name, copy, sharp_folders):
    """Portions of 1-16, 17-64 and more rows take different matrix-product kernels in bfloat16, and other ones again
    when the weights have no tiled copy; all of them follow the plain model."""
    folder, V = sharp_folders[name, "bfloat16"], TINY[name]["vocab_size"]
    runner = load_runner(folder, torch.bfloat16, num_pages=24, decode_weight_copy=copy)
    ids = seeded_ids(33, 212, V)
    want = plain_logits(folder, ids)
    runner.add_request("p")
    got, at = [], 0
    for m in (40, 17, 3, 64, 1, 16, 70, 1):
        got.append(runner.step([StepEntry("p", ids[at:at + m], list(range(m)))]).cpu()); at += m
    assert at == 212 and rel_err(torch.cat(got), want) < tol("bfloat16", name)
    runner.free_request("p")


# ---- captured decode steps ----------------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "C"])
def test_replayed_decode_graphs_equal_eager_steps(name, dtype, sharp_folders):
    """The same trace with captured decode steps and without: every replay (many per graph, with eager
    prefill steps and synchronisations between them, across block-table widths and changing batches)
    must give the eager logits."""
    folder = sharp_folders[name, dtype]
    V = TINY[name]["vocab_size"]
    eager = load_runner(folder, DT[dtype], num_pages=64)
    eager.decode_graphs = False
    graphed = load_runner(folder, DT[dtype], num_pages=64)
    graphed.GRAPH_WIDTH_MULTIPLE = 2                     # a new layout every 32 positions
    assert graphed.decode_graphs
    seqs = {r: seeded_ids(400 + i, n, V) for i, (r, n) in enumerate({"a": 150, "b": 90, "c": 120}.items())}
    pos = {r: 0 for r in seqs}
    plan = [("a", 20), ("b", 5)] + [("ab", 1)] * 30 + [("c", 33)] + [("abc", 1)] * 25 + [("free b", 0)] + [("ac", 1)] * 27
    replays = 0
    for who, n in plan:
        if who.startswith("free"):
            for r in (eager, graphed):
                r.free_request(who.split()[1])
            continue
        entries = []
        for rid in who:
            for r in (eager, graphed):
                if not r.has_request(rid):
                    r.add_request(rid)
            entries.append(StepEntry(rid, seqs[rid][pos[rid]: pos[rid] + n], [n - 1]))
            pos[rid] += n
        before = len(graphed._graphs)
        want, got = eager.step(entries).cpu(), graphed.step(entries).cpu()
        replays += n == 1 and len(graphed._graphs) == before
        if dtype == "float32":
            assert torch.equal(got, want), (who, pos)
        else:
            assert torch.allclose(got, want, rtol=0, atol=0), (who, pos)   # same kernels, same order: equal bits
    assert replays > 60 and len(graphed._graphs) >= 4
    want = plain_logits(folder, seqs["a"][: pos["a"]])[-1]
    assert rel_err(got[0], want) < tol(dtype, name)


@pytest.mark.parametrize("name", ["A", "C"])
def test_decode_rows_taken_whole_by_one_workgroup_in_the_engine(name, sharp_folders, monkeypatch):
    """The row kernel that takes a (row, kv head) pair whole in one workgroup, inside the engine: forced for every
    step of single tokens (it is chosen from 192 pairs on, which tiny models reach only with 64 requests: the second
    half of this test), eagerly and in replayed graphs, with C's window of 24 keys and its second cache group.  Every
    row is the plain model's within the configuration's bound, and the kernel is the one that ran."""
    from inferflux_amd.kernels import attention, ops
    folder, V = sharp_folders[name, "bfloat16"], TINY[name]["vocab_size"]
    used = []
    real = ops.attention_rows
    monkeypatch.setattr(ops, "attention_rows", lambda *a: (used.append(a[-2]), real(*a))[1])
    monkeypatch.setattr(attention, "ROW_WHOLE_MIN_PAIRS", 1)
    runner = load_runner(folder, torch.bfloat16, num_pages=64, max_requests=4)
    seqs = {r: seeded_ids(440 + i, n, V) for i, (r, n) in enumerate({"a": 130, "b": 47, "c": 200}.items())}
    heads = {"a": 90, "b": 7, "c": 161}
    for rid, ids in seqs.items():
        runner.add_request(rid)
        runner.step([StepEntry(rid, ids[:heads[rid]], [])])
    got = {r: [] for r in seqs}
    for k in range(39):
        live = [r for r in seqs if heads[r] + k < len(seqs[r])]
        logits = runner.step([StepEntry(r, [seqs[r][heads[r] + k]], [0]) for r in live]).float().cpu()
        for i, r in enumerate(live):
            got[r].append(logits[i].clone())
    assert used and all(w >= 1 for w in used) and runner.graph_replays > 20
    for r, rows in got.items():
        want = plain_logits(folder, seqs[r])[heads[r]: heads[r] + len(rows)]
        assert rel_err(torch.stack(rows), want) < tol("bfloat16", name), r


@pytest.mark.parametrize("which", ["tall", "narrow"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_nine_to_sixteen_rows_through_the_product_that_shares_x(name, which, sharp_folders, monkeypatch):
    """Steps of 9-16 rows in which products take the kernel that shares x through LDS, against the plain model: decode
    steps of 9-16 requests, eager and replayed, and prompt portions of 9-16 tokens.  "tall": gate/up and the head, with
    the norm's factor per row (large tall weights do by themselves; the tiny models' are made to by lowering the sizes
    from which it applies to just above their hidden size, so that o and down keep adding into the stream).  "narrow":
    o, down and q/k/v, which then leave the stream add to the norm's kernel (large weights whose tiles lie unevenly on
    the chip do by themselves; here every weight is made to)."""
    from inferflux_amd.kernels import ops
    cfg = TINY[name]
    folder, V = sharp_folders[name, "bfloat16"], cfg["vocab_size"]
    assert min(2 * cfg["intermediate_size"], V) > cfg["hidden_size"]
    if which == "tall":
        monkeypatch.setattr(ops, "WIDE_FEW_ROWS_MIN_N", cfg["hidden_size"] + 1)
        monkeypatch.setattr(ops, "WIDE_FEW_ROWS_MIN_WEIGHT", 1)
    else:
        monkeypatch.setattr(ops, "UNEVEN_TILES_MIN_WEIGHT", 1)
        lw = ops.prepare_linear(torch.zeros(cfg["hidden_size"], cfg["intermediate_size"], dtype=torch.bfloat16, device="cuda"))
        assert not ops.adds_into_stream(9, lw, torch.zeros(cfg["hidden_size"], dtype=torch.bfloat16, device="cuda"))
    used = []
    real = ops.wide_gemm
    monkeypatch.setattr(ops, "wide_gemm", lambda x, *a, **k: (used.append((x.shape[0], isinstance(x, ops.ScaledRows))), real(x, *a, **k))[1])
    runner = load_runner(folder, torch.bfloat16, num_pages=96, max_requests=16)
    seqs = {f"r{i}": seeded_ids(640 + i, 40 + 5 * i, V) for i in range(16)}
    heads = {r: 9 + (i % 8) for i, r in enumerate(seqs)}                  # prompts of 9-16 tokens, one step each
    for rid, ids in seqs.items():
        runner.add_request(rid)
        first = runner.step([StepEntry(rid, ids[:heads[rid]], list(range(heads[rid])))]).float().cpu()
        assert rel_err(first, plain_logits(folder, ids)[:heads[rid]]) < tol("bfloat16", name), rid
    got = {r: [] for r in seqs}
    for k in range(21):
        live = [r for r in seqs if int(r[1:]) < 9 or k < 3 * (16 - int(r[1:]))]           # 16 requests, one fewer every three steps, 9 at the end
        logits = runner.step([StepEntry(r, [seqs[r][heads[r] + k]], [0]) for r in live]).float().cpu()
        for i, r in enumerate(live):
            got[r].append(logits[i].clone())
    assert any(9 <= m <= 16 and (scaled or which == "narrow") for m, scaled in used) and runner.graph_replays > 5, used[-8:]
    for r, rows in got.items():
        want = plain_logits(folder, seqs[r])[heads[r]: heads[r] + len(rows)]
        assert rel_err(torch.stack(rows), want) < tol("bfloat16", name), r


def test_sixty_four_requests_decode_together(sharp_folders, monkeypatch):
    """Sixty-four requests of configuration C (3 kv heads: 192 (row, kv head) pairs, from which on a pair is taken
    whole by one workgroup) decode together after prompts of 3-60 tokens: every request's rows are the plain model's."""
    from inferflux_amd.kernels import ops
    folder, V = sharp_folders["C", "bfloat16"], TINY["C"]["vocab_size"]
    used = []
    real = ops.attention_rows
    monkeypatch.setattr(ops, "attention_rows", lambda *a: (used.append(a[-2]), real(*a))[1])
    runner = load_runner(folder, torch.bfloat16, num_pages=64 * 5, max_requests=64)
    seqs = {r: seeded_ids(1500 + r, 3 + (r * 7) % 58 + 12, V) for r in range(64)}
    for r, ids in seqs.items():
        runner.add_request(r)
    runner.step([StepEntry(r, ids[:-12], []) for r, ids in seqs.items()])          # all prompts in one step
    rows = {r: [] for r in seqs}
    for k in range(12):
        logits = runner.step([StepEntry(r, [ids[len(ids) - 12 + k]], [0]) for r, ids in seqs.items()]).float().cpu()
        for i, r in enumerate(seqs):
            rows[r].append(logits[i].clone())
    assert used and all(w >= 1 for w in used[-6:]), used[-6:]                        # decode steps of 64 rows: pairs taken whole
    worst = max(rel_err(torch.stack(rows[r]), plain_logits(folder, seqs[r])[-12:]) for r in seqs)
    assert worst < tol("bfloat16", "C"), worst
    for r in seqs:
        runner.free_request(r)
    assert runner.manager.free_pages() == [64 * 5] * 2


# ---- other toy parts: a position encoding of its own, a feed-forward with routing --------------------
def test_toy_position_encoding_and_routed_feed_forward(tmp_path):
    """Two more parts defined here and registered from outside the package: a position encoding that
    transforms q and k itself (through ``apply``, not the fused rotary kernel) and a feed-forward that
    routes each row to one of two experts.  A model built from them must agree with a plain
    computation of the same formulas and must not depend on the cutting."""
    from inferflux_amd.engine.model import Model
    from inferflux_amd.engine.runner import ModelRunner
    from inferflux_amd.parts import (FeedForward, LayerSpec, ModelPlan, ParamSpec, PartSpec, PositionEncoding,
                                     ScheduleEntry, register_part)

    H, V, nH, d = 32, 40, 2, 16

    @register_part("position", "toy_decay_scale")
    class DecayScale(PositionEncoding):
        """q is scaled by 1 + pos/100 and k by 1/(1 + pos/50): scores then depend on both positions."""
        needs_apply = True
        def __init__(self, head_dim):
            self.head_dim = head_dim
        def apply(self, q, k, positions):
            p = positions.to(torch.float32)[:, None, None]
            q = (q.float() * (1 + p / 100)).to(q.dtype)
            if k is not None:
                k = (k.float() / (1 + p / 50)).to(k.dtype)
            return q, k

    @register_part("ffn", "toy_two_experts")
    class TwoExperts(FeedForward):
        def __init__(self, name, hidden_size):
            self.name, self.H = name, hidden_size
        def param_specs(self):
            return {f"{self.name}.router.weight": ParamSpec((2, self.H), ("normal", 1.0)),
                    f"{self.name}.experts.0.weight": ParamSpec((self.H, self.H), ("normal", 0.2)),
                    f"{self.name}.experts.1.weight": ParamSpec((self.H, self.H), ("normal", 0.2))}
        def load(self, tensors):
            self.router = tensors[f"{self.name}.router.weight"]
            self.experts = [tensors[f"{self.name}.experts.{e}.weight"] for e in (0, 1)]
        def forward(self, h, ctx):
            choice = (h.float() @ self.router.float().t()).argmax(-1)          # router logits in 32-bit
            out = torch.zeros_like(h)
            for e in (0, 1):
                rows = (choice == e).nonzero().flatten()
                if rows.numel():
                    out[rows] = torch.tanh(h[rows] @ self.experts[e].t())
            return out

    p = "toy.layers.0"
    layer = LayerSpec(p, PartSpec("prenorm"), PartSpec("rmsnorm", {"name": f"{p}.n1", "eps": 1e-5}),
                      PartSpec("paged_attention", {"name": f"{p}.attn", "n_heads": nH, "n_kv_heads": 1, "head_dim": d,
                                                   "bias": True, "position": PartSpec("toy_decay_scale", {"head_dim": d})}),
                      PartSpec("rmsnorm", {"name": f"{p}.n2", "eps": 1e-5}),
                      PartSpec("toy_two_experts", {"name": f"{p}.moe"}))
    plan = ModelPlan(vocab_size=V, hidden_size=H, max_position=128,
                     embedding=PartSpec("token_embedding", {"name": "toy.embed", "vocab_size": V}),
                     layers=(layer,), schedule=(ScheduleEntry(0),),
                     final_norm=PartSpec("rmsnorm", {"name": "toy.norm", "eps": 1e-5}),
                     lm_head=PartSpec("linear_head", {"name": "toy.head", "vocab_size": V}))
    model = Model(plan=plan).init_random(5, torch.float32, "cuda")
    assert not model.graph_safe                                         # parts from outside are not replayed as graphs
    runner = ModelRunner(model, num_pages=16, max_requests=2)
    assert not runner.decode_graphs
    ids = seeded_ids(16, 50, V)
    runner.add_request("w")
    whole = runner.step([StepEntry("w", ids, list(range(50)))]).cpu()
    runner.free_request("w")
    runner.add_request("c")
    rows, q = [], 0
    for mlen in (9, 1, 1, 20, 2, 17):
        rows.append(runner.step([StepEntry("c", ids[q:q + mlen], list(range(mlen)))]).cpu()); q += mlen
    assert torch.allclose(torch.cat(rows), whole, rtol=1e-4, atol=1e-5)

    # the same formulas, plainly, from the model's own tensors
    att, moe = model.blocks[0].mixer, model.blocks[0].ffn
    x = model.embedding.table.double().cpu()[ids]
    pos = torch.arange(50, dtype=torch.float64)
    h = pm.rms_norm(x, model.blocks[0].norm_in.weight.double().cpu(), 1e-5)
    qkv = h @ att.w_qkv.rows.double().cpu().t() + att.b_qkv.double().cpu()
    qq = qkv[:, : nH * d].view(50, nH, d) * (1 + pos / 100)[:, None, None]
    kk = qkv[:, nH * d: (nH + 1) * d].view(50, 1, d) / (1 + pos / 50)[:, None, None]
    vv = qkv[:, (nH + 1) * d:].view(50, 1, d)
    x = x + pm.attention(qq, kk, vv).reshape(50, nH * d) @ att.w_o.rows.double().cpu().t()
    h = pm.rms_norm(x, model.blocks[0].norm_post.weight.double().cpu(), 1e-5)
    choice = (h @ moe.router.double().cpu().t()).argmax(-1)
    y = torch.stack([torch.tanh(h[i] @ moe.experts[int(choice[i])].double().cpu().t()) for i in range(50)])
    x = x + y
    want = pm.rms_norm(x, model.final_norm.weight.double().cpu(), 1e-5) @ model.head.weight.rows.double().cpu().t()
    assert torch.allclose(whole.double(), want, rtol=1e-3, atol=1e-4)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("page_size", [32, 64, 128])
def test_other_page_sizes(page_size, dtype, sharp_folders):
    """Pages of 32, 64 (trace_run's rounding unit) and 128 tokens: mixed steps over a pool that is used again."""
    import traces
    folder = sharp_folders["C", dtype]
    seqs = {f"r{i}": seeded_ids(500 + i, n, 777) for i, n in enumerate([70, 130, 45, 200, 64])}
    steps, expected = traces.mixed(seqs, seed=page_size)
    runner = load_runner(folder, DT[dtype], num_pages=traces.peak_tokens(steps, page_size) // page_size, page_size=page_size)
    for s in steps:
        for e in s["entries"]:
            if not runner.has_request(e["id"]):
                runner.add_request(e["id"])
        got = runner.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in s["entries"]]).cpu()
        if s["step"] in expected:
            want = torch.stack([plain_logits(folder, seqs[rid])[p] for rid, p in expected[s["step"]]])
            assert rel_err(got, want) < tol(dtype, "C"), s["step"]
        for rid in s["end"]:
            runner.free_request(rid)
        runner.manager.check()
    assert runner.manager.free_pages() == [p.num_pages for p in runner.manager.pools]


def test_prompt_portions_with_a_long_past_split_their_keys(sharp_folders, monkeypatch):
    """Portions of a prompt late in a long context: few tiles, many keys, which the tile kernel cuts into splits.
    The thresholds are lowered so that the tiny models' 250 and 380 tokens qualify."""
    from inferflux_amd.kernels import attention
    for name, value in (("TILE_SPLIT_MIN_KEYS", 64), ("TILE_SPLIT_MIN_LONGEST", 128), ("TILE_SPLIT_FEW_MIN_LONGEST", 128),
                        ("TILE_SPLIT_FEW_MIN_KEYS", 64), ("TILE_QT2_MIN_KEYS", 300), ("TILE_ORDER_MIN_ITEMS", 0)):
        monkeypatch.setattr(attention, name, value)
    calls = []
    real = attention.ops.attention_tiles
    monkeypatch.setattr(attention.ops, "attention_tiles", lambda *a, **k: (calls.append(a[14] if len(a) > 14 else 1), real(*a, **k))[1])
    for name, portions in (("A", (100, 90, 17, 43)), ("C", (150, 100, 17, 113))):
        folder = sharp_folders[name, "bfloat16"]
        runner = load_runner(folder, torch.bfloat16, num_pages=40)
        ids = seeded_ids(77, sum(portions), TINY[name]["vocab_size"])
        want = plain_logits(folder, ids)
        runner.add_request("p")
        pos = 0
        for n in portions:
            got = runner.step([StepEntry("p", ids[pos:pos + n], list(range(n)))]).cpu()
            assert rel_err(got, want[pos:pos + n]) < tol("bfloat16", name), (name, pos)
            pos += n
        runner.free_request("p")
    assert max(calls) > 1      # some portion did run in splits


ODD_SIZES = {
    # hidden width that no head count divides into, feed-forward and vocabulary that are multiples of nothing much
    "width100": dict(vocab_size=333, hidden_size=100, num_hidden_layers=2, num_attention_heads=5, num_key_value_heads=5,
                     head_dim=16, intermediate_size=90),
    # thirty-two query heads on one key head (two tiles of sixteen in the grouped kernels)
    "ratio32": dict(vocab_size=5001, hidden_size=200, num_hidden_layers=2, num_attention_heads=32, num_key_value_heads=1,
                    head_dim=48, intermediate_size=1000),
    # a head size beyond what the matrix-core attention takes: the plain kernel in both precisions
    "head256": dict(vocab_size=1111, hidden_size=136, num_hidden_layers=2, num_attention_heads=2, num_key_value_heads=1,
                    head_dim=256, intermediate_size=264),
    # seventeen heads of 80
    "heads17": dict(vocab_size=4099, hidden_size=272, num_hidden_layers=1, num_attention_heads=17, num_key_value_heads=17,
                    head_dim=80, intermediate_size=530, tie_word_embeddings=True),
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(ODD_SIZES))
def test_sizes_that_are_multiples_of_little(name, dtype, tmp_path):
    from conftest import QK_GAIN, sharpen
    from inferflux_amd.config import config_from_dict
    from inferflux_amd.weights import write_random_model
    cfg = {**TINY["A"], "tie_word_embeddings": False, **ODD_SIZES[name]}
    raw, folder = str(tmp_path / "raw"), str(tmp_path / "sharp")
    write_random_model(raw, config_from_dict(cfg), seed=5, dtype=torch.bfloat16)
    sharpen(raw, folder, 6, QK_GAIN[dtype] / 2 if name == "heads17" else QK_GAIN[dtype])   # (272 wide: scores grow with the width)
    ids = seeded_ids(3, 120, cfg["vocab_size"])
    want = plain_logits(folder, ids)
    runner = load_runner(folder, DT[dtype], num_pages=16)
    runner.add_request("a")
    got = [runner.step([StepEntry("a", ids[:70], list(range(70)))]).cpu(),
           runner.step([StepEntry("a", ids[70:87], list(range(17)))]).cpu()]        # 17 rows: one more than a tile
    got += [runner.step([StepEntry("a", [ids[p]], [0])]).cpu() for p in range(87, 120)]
    assert rel_err(torch.cat(got), want) < REL_TOL[dtype]


@pytest.mark.parametrize("seed", range(12))
def test_configurations_drawn_at_random(seed, tmp_path):
    """Configurations drawn at random (1-3 layers, head sizes of 8-128, 1-3 kv heads with 1-4 query heads each, a
    width that need not be heads x head size, odd vocabularies, with and without bias, tied head, a window on the
    upper layers; pages of 16 or 32), each run as a mix of up to four live requests in a pool so small that pages are
    used again.  float32 against the plain model at the tight bound, and bfloat16 beside float32 at bfloat16's."""
    import random
    import traces
    from conftest import QK_GAIN, sharpen
    from inferflux_amd.config import config_from_dict
    from inferflux_amd.weights import write_random_model
    rng = random.Random(4000 + seed)
    d = rng.choice([8, 16, 24, 32, 48, 64, 128])
    nKV = rng.randint(1, 3)
    nH = nKV * rng.randint(1, 4)
    window = rng.random() < 0.4
    layers = rng.randint(1, 3)
    cfg = dict(model_type="qwen2", architectures=["Qwen2ForCausalLM"], vocab_size=rng.randint(40, 2500),
               hidden_size=8 * rng.randint(3, 30), num_hidden_layers=layers, num_attention_heads=nH, num_key_value_heads=nKV,
               head_dim=d, intermediate_size=8 * rng.randint(3, 60), max_position_embeddings=512,
               rope_theta=rng.choice([1e4, 5e5, 1e6]), rms_norm_eps=rng.choice([1e-6, 1e-5, 3e-6]),
               tie_word_embeddings=rng.random() < 0.5, attention_bias=rng.random() < 0.6, use_sliding_window=window,
               sliding_window=rng.randint(5, 60), max_window_layers=rng.randint(0, layers - 1) if window else layers,
               hidden_act="silu", torch_dtype="bfloat16")
    page_size = rng.choice([16, 16, 32])
    raw = str(tmp_path / "raw")
    write_random_model(raw, config_from_dict(cfg), seed=seed, dtype=torch.bfloat16)
    seqs = {f"r{i}": seeded_ids(seed * 10 + i, rng.randint(3, 150), cfg["vocab_size"]) for i in range(6)}
    steps, expected = traces.mixed(seqs, seed=seed)
    pages = traces.peak_tokens(steps, round_to=page_size) // page_size
    for dtype in ("float32", "bfloat16"):
        folder = str(tmp_path / dtype)
        sharpen(raw, folder, 50 + seed, QK_GAIN[dtype] * min(1.0, (64 / cfg["hidden_size"]) ** 0.5))   # (scores grow with the width)
        n_pages = pages + (1 if window else 0)
        runner = load_runner(folder, DT[dtype], num_pages=n_pages, page_size=page_size, max_requests=4)
        got, want = [], []
        for st in steps:
            for e in st["entries"]:
                if not runner.has_request(e["id"]):
                    runner.add_request(e["id"])
            logits = runner.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in st["entries"]])
            if st["step"] in expected:
                got.append(logits.float().cpu())
                want += [plain_logits(folder, seqs[rid])[p] for rid, p in expected[st["step"]]]
            for rid in st["end"]:
                runner.free_request(rid)
        e = rel_err(torch.cat(got), torch.stack(want))
        print(f"random configuration {seed} {dtype}: {e:.2e}", flush=True)
        assert e < REL_TOL[dtype], (seed, dtype, e, cfg, page_size)
        runner.manager.check()
        assert runner.manager.free_pages() == [n_pages] * len(runner.manager.groups), (seed, dtype)


def test_a_toy_embedding_that_reads_positions_and_a_toy_mixer_with_narrow_values(tmp_path):
    """Two parts from outside the package that need more of the step than the built-in ones: an embedding that adds
    a learned table of absolute positions (it is given the step's context, not just the token ids), and an
    attention whose values are narrower than its keys (d = 24, dv = 8: the cache spec, the storage, the planner's
    bytes per token and the plain attention kernel all take the two widths).  Whole against cut, and against the
    formulas written out."""
    from inferflux_amd.engine.api import plan_kv_pages
    from inferflux_amd.engine.model import Model
    from inferflux_amd.engine.runner import ModelRunner
    from inferflux_amd.kernels import ops
    from inferflux_amd.parts import CacheSpec, LayerSpec, Mixer, ModelPlan, ParamSpec, PartSpec, ScheduleEntry, register_part
    from inferflux_amd.parts.base import Part

    H, V, nH, d, dv, MAXP = 40, 70, 2, 24, 8, 96

    @register_part("embedding", "toy_token_plus_position")
    class TokenPlusPosition(Part):
        def __init__(self, name, vocab_size, hidden_size, max_position):
            self.name, self.V, self.H, self.maxp = name, vocab_size, hidden_size, max_position
        def param_specs(self):
            return {f"{self.name}.tokens.weight": ParamSpec((self.V, self.H)),
                    f"{self.name}.positions.weight": ParamSpec((self.maxp, self.H), ("normal", 0.05))}
        def load(self, tensors):
            self.tokens, self.positions = tensors[f"{self.name}.tokens.weight"], tensors[f"{self.name}.positions.weight"]
        def forward(self, ctx):
            return ops.embedding(ctx.token_ids, self.tokens) + ops.embedding(ctx.positions, self.positions)

    @register_part("mixer", "toy_narrow_value_attention")
    class NarrowValues(Mixer):
        def __init__(self, name, hidden_size):
            self.name, self.H = name, hidden_size
        def cache_spec(self):
            return CacheSpec(n_kv_heads=1, head_dim=d, v_head_dim=dv)
        def param_specs(self):
            n = self.name
            return {f"{n}.q.weight": ParamSpec((nH * d, self.H), ("normal", 0.3)), f"{n}.k.weight": ParamSpec((d, self.H), ("normal", 0.3)),
                    f"{n}.v.weight": ParamSpec((dv, self.H), ("normal", 0.3)), f"{n}.o.weight": ParamSpec((self.H, nH * dv), ("normal", 0.3))}
        def load(self, tensors):
            self.wq, self.wk, self.wv, self.wo = (tensors[f"{self.name}.{p}.weight"] for p in "qkvo")
        def forward(self, h, ctx, binding):
            cache = binding.cache
            P = cache.page_size
            slots = ctx.write_slots(cache.group).long()
            k, v = h @ self.wk.t(), h @ self.wv.t()
            cache.k[slots // P, 0, slots % P] = k                          # K [page][head][offset][d]
            cache.v[slots // P, 0, :, slots % P] = v                       # V [page][head][dv][offset]
            q = (h @ self.wq.t()).view(-1, nH, d).contiguous()
            out = ops.attention_plain(q, cache.k, cache.v, ctx.row_req, ctx.positions, ctx.block_table(cache.group), None, d ** -0.5)
            return out @ self.wo.t()

    p = "toy.layers.0"
    layer = LayerSpec(p, PartSpec("prenorm"), PartSpec("rmsnorm", {"name": f"{p}.n1", "eps": 1e-5}),
                      PartSpec("toy_narrow_value_attention", {"name": f"{p}.attn"}),
                      PartSpec("rmsnorm", {"name": f"{p}.n2", "eps": 1e-5}),
                      PartSpec("swiglu", {"name": f"{p}.mlp", "intermediate_size": 56}))
    plan = ModelPlan(vocab_size=V, hidden_size=H, max_position=MAXP,
                     embedding=PartSpec("toy_token_plus_position", {"name": "toy.embed", "vocab_size": V, "max_position": MAXP}),
                     layers=(layer,), schedule=(ScheduleEntry(0),),
                     final_norm=PartSpec("rmsnorm", {"name": "toy.norm", "eps": 1e-5}),
                     lm_head=PartSpec("linear_head", {"name": "toy.head", "vocab_size": V}))
    model = Model(plan=plan).init_random(9, torch.float32, "cuda")
    runner = ModelRunner(model, num_pages=8, max_requests=2)
    cache = runner.storage.binding(0).cache
    assert tuple(cache.k.shape) == (8 + 1, 1, 16, d) and tuple(cache.v.shape) == (8 + 1, 1, dv, 16)     # (one scratch page beyond the pool)
    assert runner.storage.bytes_per_token() == (d + dv) * 4
    assert plan_kv_pages(model, 16, 16 * 5) == 5                        # (sized by tokens; the bytes only cap it)
    ids = seeded_ids(31, 60, V)
    runner.add_request("w")
    whole = runner.step([StepEntry("w", ids, list(range(60)))]).cpu()
    runner.free_request("w")
    runner.add_request("o"); runner.add_request("c")
    rows, at = [], 0
    for m in (13, 1, 2, 30, 1, 13):
        rows.append(runner.step([StepEntry("o", ids[at:at + 1], []), StepEntry("c", ids[at:at + m], list(range(m)))]).cpu()[:m])
        at += m
    assert torch.allclose(torch.cat(rows), whole, rtol=1e-4, atol=1e-5)
    # the formulas, plainly
    emb, att, blk = model.embedding, model.blocks[0].mixer, model.blocks[0]
    D = lambda t: t.double().cpu()
    x = D(emb.tokens)[ids] + D(emb.positions)[:60]
    h = pm.rms_norm(x, D(blk.norm_in.weight), 1e-5)
    q, k, v = (h @ D(att.wq).t()).view(60, nH, d), (h @ D(att.wk).t()).view(60, 1, d), (h @ D(att.wv).t()).view(60, 1, dv)
    s = torch.einsum("ihd,jd->hij", q, k[:, 0]) * d ** -0.5
    s = s.masked_fill(torch.triu(torch.ones(60, 60, dtype=torch.bool), 1), float("-inf"))
    o = torch.einsum("hij,je->ihe", torch.softmax(s, -1), v[:, 0]).reshape(60, nH * dv)
    x = x + o @ D(att.wo).t()
    h = pm.rms_norm(x, D(blk.norm_post.weight), 1e-5)
    x = x + pm.swiglu(h, D(blk.ffn.w_gate_up.rows)[0::2], D(blk.ffn.w_gate_up.rows)[1::2], D(blk.ffn.w_down.rows))
    want = pm.rms_norm(x, D(model.final_norm.weight), 1e-5) @ D(model.head.weight.rows).t()
    assert torch.allclose(whole.double(), want, rtol=1e-3, atol=1e-4)
    # the position table matters: without it the logits are others
    emb.positions.zero_()
    runner.free_request("o")
    runner.add_request("z")
    assert not torch.allclose(runner.step([StepEntry("z", ids[:10], list(range(10)))]).cpu(), whole[:10], rtol=1e-2, atol=1e-3)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("d,dv", [(16, 8), (16, 40), (32, 32)])
def test_builtin_attention_with_values_of_another_width_than_keys(d, dv, dtype):
    """The package's own attention part with value heads narrower and wider than the key heads (and, as the control,
    as wide): the plan says ``v_head_dim``, the part sizes its v and o projections and its cache by it, and such a
    layer runs on the kernels that take both widths (in bfloat16 too: the plain attention kernel, the unfused
    projection path).  Whole against cut, and against the formulas written out, rotary positions and biases included."""
    from inferflux_amd.engine.model import Model
    from inferflux_amd.engine.runner import ModelRunner
    from inferflux_amd.parts import LayerSpec, ModelPlan, PartSpec, ScheduleEntry
    H, V, nH, nKV, theta, N = 48, 90, 4, 2, 10000.0, 70
    p = "toy.layers.0"
    attn = PartSpec("paged_attention", {"name": f"{p}.attn", "n_heads": nH, "n_kv_heads": nKV, "head_dim": d, "v_head_dim": dv,
                                        "bias": True, "init_std": 0.3, "position": PartSpec("rotary", {"head_dim": d, "theta": theta})})
    layer = LayerSpec(p, PartSpec("prenorm"), PartSpec("rmsnorm", {"name": f"{p}.n1", "eps": 1e-5}), attn,
                      PartSpec("rmsnorm", {"name": f"{p}.n2", "eps": 1e-5}),
                      PartSpec("swiglu", {"name": f"{p}.mlp", "intermediate_size": 64}))
    plan = ModelPlan(vocab_size=V, hidden_size=H, max_position=128,
                     embedding=PartSpec("token_embedding", {"name": "toy.embed", "vocab_size": V}),
                     layers=(layer,), schedule=(ScheduleEntry(0),),
                     final_norm=PartSpec("rmsnorm", {"name": "toy.norm", "eps": 1e-5}),
                     lm_head=PartSpec("linear_head", {"name": "toy.head", "vocab_size": V}))
    model = Model(plan=plan).init_random(12, DT[dtype], "cuda")
    specs = model.param_specs()
    assert specs[f"{p}.attn.v_proj.weight"].shape == (nKV * dv, H) and specs[f"{p}.attn.o_proj.weight"].shape == (H, nH * dv)
    runner = ModelRunner(model, num_pages=10, max_requests=2)
    cache = runner.storage.binding(0).cache
    assert tuple(cache.k.shape[1:]) == (nKV, 16, d) and tuple(cache.v.shape[1:]) == (nKV, dv, 16)
    ids = seeded_ids(33, N, V)
    runner.add_request("w")
    whole = runner.step([StepEntry("w", ids, list(range(N)))]).cpu()
    runner.free_request("w")
    runner.add_request("o"); runner.add_request("c")
    rows, at = [], 0
    for m in (17, 1, 2, 30, 1, 19):
        rows.append(runner.step([StepEntry("o", ids[at:at + 1], []), StepEntry("c", ids[at:at + m], list(range(m)))]).cpu()[:m])
        at += m
    cut = torch.cat(rows)
    # the formulas, plainly, from the tensors the parts hold
    att, blk = model.blocks[0].mixer, model.blocks[0]
    D = lambda t: t.double().cpu()
    wqkv, bqkv = D(att.w_qkv.rows), D(att.b_qkv)
    x = D(model.embedding.table)[ids]
    h = pm.rms_norm(x, D(blk.norm_in.weight), 1e-5)
    qkv = h @ wqkv.t() + bqkv
    q = pm.rope_split_half(qkv[:, :nH * d].reshape(N, nH, d), list(range(N)), theta)
    k = pm.rope_split_half(qkv[:, nH * d:(nH + nKV) * d].reshape(N, nKV, d), list(range(N)), theta)
    v = qkv[:, (nH + nKV) * d:].reshape(N, nKV, dv)
    s = torch.einsum("ihd,jhd->hij", q, k.repeat_interleave(nH // nKV, dim=1)) * d ** -0.5
    s = s.masked_fill(torch.triu(torch.ones(N, N, dtype=torch.bool), 1), float("-inf"))
    o = torch.einsum("hij,jhe->ihe", torch.softmax(s, -1), v.repeat_interleave(nH // nKV, dim=1)).reshape(N, nH * dv)
    x = x + o @ D(att.w_o.rows).t()
    h = pm.rms_norm(x, D(blk.norm_post.weight), 1e-5)
    x = x + pm.swiglu(h, D(blk.ffn.w_gate_up.rows)[0::2], D(blk.ffn.w_gate_up.rows)[1::2], D(blk.ffn.w_down.rows))
    want = pm.rms_norm(x, D(model.final_norm.weight), 1e-5) @ D(model.head.weight.rows).t()
    if dtype == "float32":
        assert torch.allclose(cut, whole, rtol=1e-4, atol=1e-5)
        assert rel_err(whole, want) < REL_TOL["float32"]
    else:
        assert rel_err(cut, want) < 3e-2 and rel_err(whole, want) < 3e-2
    assert runner.manager.free_pages() == [10 - 5 - 1]          # "c" holds 70 tokens, "o" one


def test_a_toy_block_with_four_norms_and_no_feed_forward():
    """An arrangement from outside the package that the built-in one does not cover: pre-norm, attention, a norm on
    the attention's output before the add, a norm on the skip path, and no feed-forward at all; the two further
    norms come from the layer spec's named extras.  It is registered, built and stepped; whole equals cut; and
    the formulas written out."""
    from inferflux_amd.engine.model import Model
    from inferflux_amd.engine.runner import ModelRunner
    from inferflux_amd.parts import Block, LayerSpec, ModelPlan, PartSpec, ScheduleEntry, build_part, register_part

    H, V, nH, d = 48, 80, 3, 16

    @register_part("block", "toy_sandwich_without_ffn")
    class Sandwich(Block):
        def __init__(self, layer, hidden_size):
            assert layer.ffn is None and layer.norm_post is None
            self.norm_in = build_part("norm", layer.norm_in, hidden_size=hidden_size)
            self.mixer = build_part("mixer", layer.mixer, hidden_size=hidden_size)
            self.norm_out = build_part(*layer.extra_part("norm_out"), hidden_size=hidden_size)
            self.norm_skip = build_part(*layer.extra_part("norm_skip"), hidden_size=hidden_size)
        def children(self):
            return (self.norm_in, self.mixer, self.norm_out, self.norm_skip)
        def forward(self, residual, pending, ctx, binding):
            h = self.norm_in.forward(residual, pending, ctx.act_dtype)            # (adds what the block before left pending)
            delta = self.mixer.forward(h, ctx, binding).float()
            normed = self.norm_out.forward(delta, None, torch.float32)            # a norm on the sub-block's output
            skip = self.norm_skip.forward(residual.clone(), None, torch.float32)  # and one on the skip path
            residual.copy_(skip)
            return residual, normed.to(ctx.act_dtype)

    def layer(i):
        p = f"toy.layers.{i}"
        return LayerSpec(p, PartSpec("toy_sandwich_without_ffn"), PartSpec("rmsnorm", {"name": f"{p}.n_in", "eps": 1e-5}),
                         PartSpec("paged_attention", {"name": f"{p}.attn", "n_heads": nH, "n_kv_heads": 1, "head_dim": d, "bias": False,
                                                      "position": PartSpec("rotary", {"head_dim": d, "theta": 100.0})}),
                         extra=(("norm_out", "norm", PartSpec("rmsnorm", {"name": f"{p}.n_out", "eps": 1e-5})),
                                ("norm_skip", "norm", PartSpec("rmsnorm", {"name": f"{p}.n_skip", "eps": 1e-4}))))

    plan = ModelPlan(vocab_size=V, hidden_size=H, max_position=128,
                     embedding=PartSpec("token_embedding", {"name": "toy.embed", "vocab_size": V}),
                     layers=(layer(0), layer(1)), schedule=(ScheduleEntry(0), ScheduleEntry(1)),
                     final_norm=PartSpec("rmsnorm", {"name": "toy.norm", "eps": 1e-5}),
                     lm_head=PartSpec("linear_head", {"name": "toy.head", "vocab_size": V}))
    with pytest.raises(KeyError, match="no extra part named 'nope'"):
        plan.layers[0].extra_part("nope")
    model = Model(plan=plan).init_random(12, torch.float32, "cuda")
    names = set(model.param_specs())
    assert {"toy.layers.0.n_out.weight", "toy.layers.1.n_skip.weight"} <= names and not any(".mlp." in n for n in names)
    runner = ModelRunner(model, num_pages=8, max_requests=2)
    ids = seeded_ids(41, 50, V)
    runner.add_request("w")
    whole = runner.step([StepEntry("w", ids, list(range(50)))]).cpu()
    runner.free_request("w")
    runner.add_request("c")
    rows, at = [], 0
    for m in (20, 1, 2, 26, 1):
        rows.append(runner.step([StepEntry("c", ids[at:at + m], list(range(m)))]).cpu()); at += m
    assert torch.allclose(torch.cat(rows), whole, rtol=1e-4, atol=1e-5)
    D = lambda t: t.double().cpu()
    x, pending = D(model.embedding.table)[ids], 0.0
    for b in model.blocks:
        x = x + pending
        h = pm.rms_norm(x, D(b.norm_in.weight), 1e-5)
        att = b.mixer
        qkv = h @ D(att.w_qkv.rows).t()
        q, k, v = qkv[:, :nH * d].view(50, nH, d), qkv[:, nH * d:(nH + 1) * d].view(50, 1, d), qkv[:, (nH + 1) * d:].view(50, 1, d)
        pos = list(range(50))
        q, k = pm.rope_split_half(q, pos, 100.0), pm.rope_split_half(k, pos, 100.0)
        delta = pm.attention(q, k, v).reshape(50, nH * d) @ D(att.w_o.rows).t()
        pending = pm.rms_norm(delta, D(b.norm_out.weight), 1e-5)
        x = pm.rms_norm(x, D(b.norm_skip.weight), 1e-4)
    want = pm.rms_norm(x + pending, D(model.final_norm.weight), 1e-5) @ D(model.head.weight.rows).t()
    assert torch.allclose(whole.double(), want, rtol=1e-3, atol=1e-4)
    # the built-in arrangement refuses a layer it cannot be
    with pytest.raises(ValueError, match="no more and no less"):
        build_part("block", PartSpec("prenorm"), layer=plan.layers[0], hidden_size=H)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_shrinking_batch_replays_few_layouts(dtype, sharp_folders):
    """Seven requests decode and leave one by one.  A captured decode step is filled up to the next of a few batch
    sizes with rows that stand for nobody (they write to a scratch page outside the pool), so the batch passes
    through sizes 7..1 on three captured layouts (8, 4, 2; 1 alone makes a fourth) instead of seven; every step's
    logits are those of the same steps run eagerly without any such rows, bit for bit."""
    folder, V = sharp_folders["C", dtype], TINY["C"]["vocab_size"]
    eager = load_runner(folder, DT[dtype], num_pages=40, max_requests=8)
    eager.decode_graphs = False
    graphed = load_runner(folder, DT[dtype], num_pages=40, max_requests=8)
    seqs = {r: seeded_ids(700 + i, 30 + 5 * i, V) for i, r in enumerate("abcdefg")}
    at = {}
    for rid, ids in seqs.items():
        for r in (eager, graphed):
            r.add_request(rid)
            r.step([StepEntry(rid, ids[:20], [])])
        at[rid] = 20
    live = list(seqs)
    while live:
        for _ in range(3):
            entries = [StepEntry(r, [seqs[r][at[r]]], [0]) for r in live]
            want, got = eager.step(entries).cpu(), graphed.step(entries).cpu()
            assert got.shape == (len(live), V) and torch.equal(got, want), (len(live), at)
            for r in live:
                at[r] += 1
        gone = live.pop(0)
        for r in (eager, graphed):
            r.free_request(gone)
            r.manager.check()
    assert graphed.graph_captures == 4 and graphed.graph_replays == 21 - 4
    assert sorted(k[0] for k in graphed._graphs) == [1, 2, 4, 8]
    assert graphed.manager.free_pages() == eager.manager.free_pages() == [40, 40]
    # the scratch page lies beyond every pool: no block table ever names it
    assert graphed.storage.scratch_pages == [40, 40] and graphed.storage.binding(0).cache.k.shape[0] == 41
