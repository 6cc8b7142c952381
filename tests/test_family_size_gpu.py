"""The kernels at the sizes of the model family.  First two layers of the Qwen2.5-7B shape (hidden 3584, 28 query
heads on 4 kv heads of 128, feed-forward 18944, vocabulary 152064): the bfloat16 engine against the float32 engine
on the same weights under several cuttings, and the float32 engine bit-equal to itself.  Then one layer at each of
the 7B, 3B, 14B, 0.5B, 1.5B, 32B and 72B shapes, written as a folder by the test itself, against the plain model in float64
on the CPU, in both precisions and three cuttings."""
import pytest
import torch

from conftest import rel_err, seeded_ids

pytestmark = pytest.mark.gpu

SHAPE = dict(model_type="qwen2", architectures=["Qwen2ForCausalLM"], vocab_size=152064, hidden_size=3584,
             num_hidden_layers=2, num_attention_heads=28, num_key_value_heads=4, head_dim=128,
             intermediate_size=18944, max_position_embeddings=4096, rope_theta=1000000.0, rms_norm_eps=1e-6,
             tie_word_embeddings=False, attention_bias=True)


@pytest.fixture(scope="module")
def runners():
    from inferflux_amd.config import config_from_dict
    from inferflux_amd.engine.model import Model
    from inferflux_amd.engine.runner import ModelRunner
    cfg = config_from_dict(SHAPE)
    out = {}
    for name, dt in (("float32", torch.float32), ("bfloat16", torch.bfloat16)):
        model = Model(cfg).init_random(21, dt, torch.device("cuda", 0))
        # at this width N(0, 0.02) weights already give scores of standard deviation 1.4: no sharpening needed
        out[name] = ModelRunner(model, num_pages=96, max_requests=4)
    return out


def run(runner, steps):
    from inferflux_amd.engine.context import StepEntry
    rows = {}
    for entries, ends in steps:
        for rid, toks, want in entries:
            if not runner.has_request(rid):
                runner.add_request(rid)
        start = {rid: runner.length(rid) for rid, _, _ in entries}
        logits = runner.step([StepEntry(rid, toks, want) for rid, toks, want in entries]).cpu()
        i = 0
        for rid, toks, want in entries:
            for w in want:
                rows[rid, start[rid] + w] = logits[i]
                i += 1
        for rid in ends:
            runner.free_request(rid)
    return rows


def test_bfloat16_engine_follows_the_float32_engine_at_7b_layer_sizes(runners):
    a, b = seeded_ids(31, 400, SHAPE["vocab_size"]), seeded_ids(32, 150, SHAPE["vocab_size"])
    tail = list(range(360, 400))
    whole = [([("a", a, tail)], ["a"])]
    cut = [([("a", a[:330], [])], []), ([("b", b[:100], [99])], [])]
    cut += [([("a", a[330:370], list(range(30, 40))), ("b", [b[100]], [0])], [])]               # a portion beside a decode token
    cut += [([("a", [a[p]], [0]), ("b", [b[p - 269]], [0])], []) for p in range(370, 400)]      # decode steps (replayed graphs)
    cut[-1] = (cut[-1][0], ["a", "b"])
    ref_whole, ref_cut = run(runners["float32"], whole), run(runners["float32"], cut)
    for key, v in ref_cut.items():
        if key[0] == "a":
            assert torch.equal(v, ref_whole[key]), key            # float32: bit-equal under every cutting
    got_whole, got_cut = run(runners["bfloat16"], whole), run(runners["bfloat16"], cut)
    for got, ref in ((got_whole, ref_whole), (got_cut, ref_cut)):
        assert set(got) == set(ref)
        keys = sorted(got)
        e = rel_err(torch.stack([got[k] for k in keys]), torch.stack([ref[k] for k in keys]))
        assert e < 2.4e-2, e             # measured 1.58e-2 (two layers; against the float32 engine)
    assert all(r.manager.free_pages() == [96] for r in runners.values())


# ---- one layer at each family shape against the plain model ----------------------------------------------------
# The layer shapes of Qwen2.5-7B, -3B and -14B (query : kv heads 7:1, 8:1, 5:1 at head size 128; feed-forward
# widths 18,944 / 11,008 / 13,824; the 152,064- and 151,936-row vocabularies) and of the small members -0.5B (head
# size 64, width 896 = 7 x 128) and -1.5B (6:1), one layer each and a tied head to keep the folders small.  The oracle is the plain implementation in float32 on the CPU, which reads the folder
# with the safetensors package: gate/up of 37,888 x 3,584, down with K = 18,944 and the head meet something that
# is not the engine here.
FAMILY = {
    "7B": dict(hidden_size=3584, num_attention_heads=28, num_key_value_heads=4, intermediate_size=18944, vocab_size=152064,
               rms_norm_eps=1e-6),
    "3B": dict(hidden_size=2048, num_attention_heads=16, num_key_value_heads=2, intermediate_size=11008, vocab_size=151936,
               rms_norm_eps=1e-6),
    "14B": dict(hidden_size=5120, num_attention_heads=40, num_key_value_heads=8, intermediate_size=13824, vocab_size=152064,
                rms_norm_eps=1e-5),
    # the small members: head size 64 on a width of 7 x 128, and 6 query heads to a kv head
    "0.5B": dict(hidden_size=896, num_attention_heads=14, num_key_value_heads=2, intermediate_size=4864, vocab_size=151936,
                 rms_norm_eps=1e-6, head_dim=64),
    "1.5B": dict(hidden_size=1536, num_attention_heads=12, num_key_value_heads=2, intermediate_size=8960, vocab_size=151936,
                 rms_norm_eps=1e-6),
    # the large members: feed-forward widths of 27,648 and 29,568 (= 2^7 x 231), a width of 8,192, 64 query heads
    "32B": dict(hidden_size=5120, num_attention_heads=40, num_key_value_heads=8, intermediate_size=27648, vocab_size=152064,
                rms_norm_eps=1e-5),
    "72B": dict(hidden_size=8192, num_attention_heads=64, num_key_value_heads=8, intermediate_size=29568, vocab_size=152064,
                rms_norm_eps=1e-5),
}
N_TOKENS = 130
# Largest difference to the plain model's (float64) logits over the largest logit.  Measured: float32 7.0e-6 / 4.7e-6 /
# 1.04e-5 at the 7B / 3B / 14B shapes, the same under every cutting (sums of up to 18,944 products in float32);
# bfloat16 1.72e-2 / 1.38e-2 / 2.08e-2 whole and by single rows, 1.32e-2 / 1.09e-2 / 1.54e-2 in portions of 17; at the 0.5B and
# 1.5B shapes float32 2.5e-6 / 3.8e-6 and bfloat16 8.9e-3 / 1.32e-2; at the 32B and 72B shapes float32 1.21e-5 / 1.38e-5
# and bfloat16 2.06e-2 / 2.32e-2.
# The bounds are those figures and half as much again (float32: the tiny configurations' 2e-5).
FAMILY_TOL = {"float32": 2e-5, "bfloat16": {"7B": 2.6e-2, "3B": 2.1e-2, "14B": 3.1e-2, "0.5B": 1.35e-2, "1.5B": 2.0e-2,
                                             "32B": 3.1e-2, "72B": 3.5e-2}}


def _rotate_pairs(w, steps, theta):
    """``w`` [d] rotated as the rotary encoding rotates a vector at position ``steps`` (which may be negative): pair p
    joins elements p and p + d/2 and turns by steps * theta^(-2p/d)."""
    d = w.shape[0]
    half = d // 2
    ang = steps * torch.pow(torch.tensor(theta, dtype=torch.float64), -2.0 * torch.arange(half, dtype=torch.float64) / d)
    x0, x1 = w[:half].double(), w[half:].double()
    return torch.cat([x0 * torch.cos(ang) - x1 * torch.sin(ang), x0 * torch.sin(ang) + x1 * torch.cos(ang)])


def _write_family_folder(folder, name, max_position=4096, distances=None):
    """config.json and model.safetensors under the Hugging Face tensor names, made here (not by the package's
    random-weights mode): N(0, 0.02) matrices with q/k doubled so that attention is peaked, norm weights around 1,
    biases of a size that matters; bfloat16-representable, so both precisions read the same numbers.

    ``distances`` (one per query head) makes every head look one way: the key bias of a kv head is a fixed vector w
    and the query bias of head h is w turned back by distances[h] positions and enlarged, so that after the rotary
    encoding a query's score is largest, by 8 and more, for the key exactly distances[h] positions behind it (the
    q/k matrices are made small beside the biases).  Each head then returns nearly the value of one far token, which
    differs from token to token: a key missed, a page or an offset wrong, a split dropped changes the logits by as
    much as they are large, at any context length, where random weights would average over thousands of keys."""
    import json
    import os
    from safetensors.torch import save_file
    shape = dict({"head_dim": 128}, **FAMILY[name])
    cfg = dict(model_type="qwen2", architectures=["Qwen2ForCausalLM"], num_hidden_layers=1,
               max_position_embeddings=max_position, rope_theta=1000000.0, tie_word_embeddings=True, attention_bias=True,
               hidden_act="silu", torch_dtype="bfloat16", **shape)
    H, nH, nKV, I, V, d = (shape["hidden_size"], shape["num_attention_heads"], shape["num_key_value_heads"],
                           shape["intermediate_size"], shape["vocab_size"], shape["head_dim"])
    g = torch.Generator(device="cuda").manual_seed(1000 + H)

    def normal(*size, std=0.02):
        return (torch.randn(size, generator=g, device="cuda") * std).to(torch.bfloat16).cpu()

    p = "model.layers.0"
    t = {"model.embed_tokens.weight": normal(V, H), "model.norm.weight": (1 + normal(H, std=0.2).float()).to(torch.bfloat16),
         f"{p}.input_layernorm.weight": (1 + normal(H, std=0.2).float()).to(torch.bfloat16),
         f"{p}.post_attention_layernorm.weight": (1 + normal(H, std=0.2).float()).to(torch.bfloat16),
         f"{p}.self_attn.q_proj.weight": normal(nH * d, H, std=0.04), f"{p}.self_attn.k_proj.weight": normal(nKV * d, H, std=0.04),
         f"{p}.self_attn.v_proj.weight": normal(nKV * d, H), f"{p}.self_attn.o_proj.weight": normal(H, nH * d),
         f"{p}.self_attn.q_proj.bias": normal(nH * d, std=0.2), f"{p}.self_attn.k_proj.bias": normal(nKV * d, std=0.2),
         f"{p}.self_attn.v_proj.bias": normal(nKV * d, std=0.2),
         f"{p}.mlp.gate_proj.weight": normal(I, H, std=0.04), f"{p}.mlp.up_proj.weight": normal(I, H, std=0.04),
         f"{p}.mlp.down_proj.weight": normal(H, I)}
    if distances is not None:
        assert len(distances) == nH
        gq = torch.Generator().manual_seed(77)
        t[f"{p}.self_attn.q_proj.weight"] = normal(nH * d, H, std=0.005)
        t[f"{p}.self_attn.k_proj.weight"] = normal(nKV * d, H, std=0.005)
        phase = torch.rand(nKV, d // 2, generator=gq, dtype=torch.float64) * 6.283185307179586
        # pair p has length 4 * 0.8^(p/2): the fast pairs, which tell neighbouring positions apart, weigh most, and the
        # score's peak (about 50) stands 9 above every other key up to 33,000 positions away
        length = 4.0 * torch.pow(torch.tensor(0.8, dtype=torch.float64), torch.arange(d // 2, dtype=torch.float64) / 2)
        w = torch.cat([length * torch.cos(phase), length * torch.sin(phase)], dim=1)     # [nKV, d]
        bq = torch.stack([7.0 * _rotate_pairs(w[h // (nH // nKV)], -float(distances[h]), cfg["rope_theta"]) for h in range(nH)])
        t[f"{p}.self_attn.k_proj.bias"] = w.reshape(-1).to(torch.bfloat16)
        t[f"{p}.self_attn.q_proj.bias"] = bq.reshape(-1).to(torch.bfloat16)
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file(t, os.path.join(folder, "model.safetensors"))
    return cfg


# One distance per query head of the 7B shape (28): page edges (15-17), the row kernel's splits (127-129), portions of
# 2,048, and keys tens of thousands of positions back.  A row that cannot reach a head's distance spreads that head's
# attention over keys whose scores nearly tie, where float32's rounding of the rotation angles alone moves the logits
# by 5e-4: every list is for rows that reach all of its distances.
DISTANCES = {
    "near": [0, 1, 2, 3, 5, 8, 15, 16, 17, 31, 32, 33, 47, 48, 63, 64, 65, 79, 80, 95, 96, 100, 111, 127, 128, 129, 144, 160],
    "far16": [0, 1, 15, 16, 17, 63, 64, 127, 128, 129, 255, 256, 511, 1023, 1024, 2047, 2048, 2049, 3000, 4095, 4096, 6000,
              8191, 8192, 10000, 12345, 15000, 16000],
    "far32": [0, 1, 16, 17, 127, 128, 129, 511, 1024, 2047, 2048, 2049, 4095, 4096, 8191, 8192, 12345, 16383, 16384, 16385,
              20000, 24000, 24575, 24576, 28000, 30000, 31000, 31900],
}
_PLAIN = {}
# The bfloat16 engine against the plain model on these folders (rows that reach every distance): 6.2e-3 to 6.9e-3
# whole, cut, mixed and at 16,384 and 32,000 tokens; the bound is that and half as much again.
DISTANCE_TOL_BF16 = 1.05e-2


class _DistanceFolders(dict):
    """key of DISTANCES -> a folder with one layer of the 7B shape whose heads look those distances back (written
    when first asked for)."""

    def __init__(self, factory):
        super().__init__()
        self.factory = factory

    def __missing__(self, key):
        self[key] = str(self.factory.mktemp(f"distance_{key}"))
        _write_family_folder(self[key], "7B", max_position=32768, distances=DISTANCES[key])
        return self[key]


@pytest.fixture(scope="module")
def distance_folders(tmp_path_factory):
    yield _DistanceFolders(tmp_path_factory)
    _PLAIN.clear()           # (the plain model's float64 weights of the folder asked for last: 6 GB, so one at a time)


def plain_rows(folder, ids, rows, angle_dtype=torch.float32):
    """The plain model's logits (float64, on the CPU) at ``rows`` of the sequence ``ids`` for a one-layer folder.  The
    rotation angles are formed in 32 bits, as the reference and the engine form them: at positions of thousands that
    rounding moves logits by more than everything else a 32-bit implementation rounds (at 16,384 tokens the float32
    engine is 3.5e-6 from this oracle at every row and up to 1.1e-4 from one with exact angles)."""
    import plain_model as pm
    if folder not in _PLAIN:
        _PLAIN.clear()
        _PLAIN[folder] = pm.load_folder(folder, torch.float64)
    cfg, W = _PLAIN[folder]
    return pm.forward_rows_one_layer(cfg, W, ids, rows, angle_dtype)


def test_distance_heads_look_where_they_are_told(distance_folders):
    """The construction itself, on the plain model's parts: with the written biases a query's largest score is at its
    head's distance, 8 and more above every other key's."""
    import math
    import plain_model as pm
    from safetensors.torch import load_file
    t = load_file(distance_folders["far32"] + "/model.safetensors")
    d, theta, n = 128, 1000000.0, 33000
    bq = t["model.layers.0.self_attn.q_proj.bias"].double().view(28, d)
    bk = t["model.layers.0.self_attn.k_proj.bias"].double().view(4, d)
    k = pm.rope_split_half(bk[None].expand(n, 4, d).clone(), list(range(n)), theta)
    q = pm.rope_split_half(bq[None], [n - 1], theta)[0]
    for h, dist in enumerate(DISTANCES["far32"]):
        s = (k[:, h // 7, :] @ q[h]) / math.sqrt(d)
        assert int(s.argmax()) == n - 1 - dist and float(s.max() - s[torch.arange(n) != n - 1 - dist].max()) > 8.0, (h, dist)


@pytest.mark.parametrize("context", [16384, 32000])
def test_long_contexts_at_the_7b_layer_shape(context, distance_folders):
    """A prompt of 16,384 and of 32,000 tokens through one layer of the 7B shape in portions of 2,048, then eight single
    tokens: the last 24 rows against the plain model evaluated for those rows only, in float32 and in bfloat16.  The
    heads look fixed distances back (to the portion's own rows, to earlier portions, to the first page), so the tile
    kernels behind long pasts with their key splits, the row kernel's splits beyond 16,384 keys and the decode steps'
    block-table widths all have to find single keys."""
    from inferflux_amd.engine.api import load_runner
    from inferflux_amd.engine.context import StepEntry
    folder = distance_folders["far16" if context <= 16384 else "far32"]
    N = context + 8
    ids = seeded_ids(41 + context, N, FAMILY["7B"]["vocab_size"])
    rows = list(range(context - 16, N))
    want = plain_rows(folder, ids, rows)
    assert torch.isfinite(want).all() and float(want.abs().max()) > 1.0
    for dtype, dt in (("float32", torch.float32), ("bfloat16", torch.bfloat16)):
        runner = load_runner(folder, dt, num_pages=N // 16 + 2, max_requests=2)
        runner.add_request("a")
        got, pos = [], 0
        while pos < context:
            n = min(2048, context - pos)
            logits = runner.step([StepEntry("a", ids[pos:pos + n], [r - pos for r in rows if pos <= r < pos + n])])
            got.append(logits.float().cpu())
            pos += n
        for p in range(context, N):
            got.append(runner.step([StepEntry("a", [ids[p]], [0])]).float().cpu().clone())
        runner.free_request("a")
        assert runner.manager.free_pages() == [N // 16 + 2]
        e = rel_err(torch.cat(got), want)
        print(f"7B layer, context {context}, {dtype}: {e:.2e}", flush=True)
        assert e < (FAMILY_TOL["float32"] if dtype == "float32" else DISTANCE_TOL_BF16), (context, dtype, e)
        del runner
        torch.cuda.empty_cache()


@pytest.mark.parametrize("name", list(FAMILY))
def test_one_layer_of_each_family_shape_against_the_plain_model(name, tmp_path):
    import plain_model as pm
    from inferflux_amd.engine.api import load_runner
    from inferflux_amd.engine.context import StepEntry
    folder = str(tmp_path / name)
    cfg = _write_family_folder(folder, name)
    ids = seeded_ids(77, N_TOKENS, cfg["vocab_size"])
    plain_cfg, W = pm.load_folder(folder, torch.float64)
    want = pm.forward(plain_cfg, W, ids)                                   # [130, V] float64, on the CPU
    del W
    assert torch.isfinite(want).all() and float(want.abs().max()) > 1.0

    def cuttings(runner):
        out = {}
        runner.add_request("w")
        out["whole"] = runner.step([StepEntry("w", ids, list(range(N_TOKENS)))]).cpu()
        runner.free_request("w")
        runner.add_request("p")
        rows = [runner.step([StepEntry("p", ids[a:a + 17], list(range(len(ids[a:a + 17]))))]).cpu() for a in range(0, N_TOKENS, 17)]
        out["17 rows"] = torch.cat(rows)
        runner.free_request("p")
        runner.add_request("d")
        rows = [runner.step([StepEntry("d", ids[:98], list(range(98)))]).cpu()]
        rows += [runner.step([StepEntry("d", [ids[q]], [0])]).cpu().clone() for q in range(98, N_TOKENS)]
        out["single rows"] = torch.cat(rows)
        runner.free_request("d")
        assert runner.manager.free_pages() == [16]
        return out

    for dtype, dt in (("float32", torch.float32), ("bfloat16", torch.bfloat16)):
        runner = load_runner(folder, dt, num_pages=16, max_requests=2)
        got = cuttings(runner)
        errs = {k: rel_err(v, want) for k, v in got.items()}
        print(f"family {name} {dtype}: " + ", ".join(f"{k} {e:.2e}" for k, e in errs.items()), flush=True)
        tol = FAMILY_TOL[dtype] if dtype == "float32" else FAMILY_TOL[dtype][name]
        assert max(errs.values()) < tol, (name, dtype, errs)
        if dtype == "float32":
            assert torch.equal(got["whole"], got["17 rows"]) and torch.equal(got["whole"], got["single rows"])
        assert (got["whole"].argmax(-1) == want.argmax(-1)).float().mean() > (0.999 if dtype == "float32" else 0.9)
        del runner, got
        torch.cuda.empty_cache()


@pytest.mark.parametrize("page_size", [16, 128])
def test_portions_behind_long_pasts_at_the_7b_layer_shape(page_size, monkeypatch, distance_folders):
    """A sequence of 3,000 tokens through one layer of the 7B shape in portions whose pasts grow to 2,364 keys: the
    tile kernels then run with tiles of 64 and of 128 rows, their keys whole and in splits of several lengths, their
    workgroups in the balanced order.  The oracle is the plain model (float64, on the CPU, from a folder this test
    wrote, its heads looking fixed distances back): the float32 engine within 2e-5 of it, every cutting of the bfloat16
    engine within the bound of the shape.  Pages of 16 tokens and of 128 (larger than a tile of 64 keys)."""
    from inferflux_amd.engine.api import load_runner
    from inferflux_amd.engine.context import StepEntry
    from inferflux_amd.kernels import attention
    folder = distance_folders["near"]
    N, last = 3000, 24
    ids = seeded_ids(5, N, SHAPE["vocab_size"])
    cuttings = ([N], [700, 1100, 64, 500, 636], [1024, 1024, 952], [256] * 11 + [184], [2560, 128, 312])
    wanted = sorted({sum(c[:i + 1]) - 1 - k for c in cuttings for i in range(len(c)) for k in range(min(last, c[i]))})
    want = plain_rows(folder, ids, wanted)
    tilings = set()
    real = attention.choose_tiling
    monkeypatch.setattr(attention, "choose_tiling", lambda *a, **k: (tilings.add(real(*a, **k)), real(*a, **k))[1])

    def run(dtype, cuts):
        runner = load_runner(folder, dtype, num_pages=N // page_size + 2, page_size=page_size, max_requests=2)
        runner.add_request("a")
        rows, pos = {}, 0
        for n in cuts:
            want_here = [p - pos for p in wanted if pos <= p < pos + n]
            logits = runner.step([StepEntry("a", ids[pos:pos + n], want_here)]).float().cpu()
            rows.update({pos + w: logits[i] for i, w in enumerate(want_here)})
            pos += n
        runner.free_request("a")
        assert runner.manager.free_pages() == [N // page_size + 2]
        return torch.stack([rows[p] for p in wanted])

    e = rel_err(run(torch.float32, [N]), want)
    print(f"7B layer, 3,000 tokens whole, float32 against the plain model: {e:.2e}", flush=True)
    assert e < FAMILY_TOL["float32"], e
    for cuts in cuttings:
        e = rel_err(run(torch.bfloat16, cuts), want)
        print(f"7B layer, 3,000 tokens in {len(cuts)} portions, bfloat16 against the plain model: {e:.2e}", flush=True)
        assert e < DISTANCE_TOL_BF16, (cuts, e)
    assert {t[0] for t in tilings} == {1, 2} and len({t[1] for t in tilings}) >= 3, tilings


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_mixed_requests_at_the_7b_layer_shape(seed, distance_folders):
    """Five requests of 200-900 tokens through one layer of the 7B shape, up to four live at a time, in portions of 2-600
    tokens beside single decoded tokens, in a pool so small that pages are used again: steps of 1-16, 17-64, 65-128
    and more rows meet every product kernel (the streaming ones, the one that shares x through LDS up to 128 rows,
    the library whole and in slices of K) and both attention kernels in one batch.  The oracle is the plain model
    (float64, on the CPU; heads that look fixed distances of up to 160 positions back) on 250 of the rows that reach so
    far back, drawn from every request: the float32 engine, which runs each request whole, within 2e-5 of it, the bfloat16 engine's mixed
    steps within the bound of the shape; and all rows of the bfloat16 engine against the float32 engine's."""
    import random
    import traces
    from inferflux_amd.engine.api import load_runner
    from inferflux_amd.engine.context import StepEntry
    folder = distance_folders["near"]
    rng = random.Random(70 + seed)
    seqs = {f"r{i}": seeded_ids(900 + 10 * seed + i, rng.randint(200, 900), SHAPE["vocab_size"]) for i in range(5)}
    steps, expected = traces.mixed(seqs, seed=seed, chunk_sizes=(2, 9, 17, 40, 70, 100, 128, 129, 300, 600))
    rows_per_step = sorted({sum(len(e["tokens"]) for e in st["entries"]) for st in steps})
    assert rows_per_step[0] <= 16 and any(64 < n <= 128 for n in rows_per_step) and rows_per_step[-1] > 256, rows_per_step
    every = [(step, i, rid, p) for step, rows in expected.items() for i, (rid, p) in enumerate(rows) if p >= max(DISTANCES["near"])]
    sample = sorted(rng.sample(every, 250))
    plain = {}
    for rid, ids in seqs.items():
        ps = sorted({p for _, _, r, p in sample if r == rid})
        plain.update({(rid, p): row for p, row in zip(ps, plain_rows(folder, ids, ps))})
    ref_runner = load_runner(folder, torch.float32, num_pages=60, max_requests=2)
    ref = {}
    for rid, ids in seqs.items():
        ref_runner.add_request(rid)
        ref[rid] = ref_runner.step([StepEntry(rid, ids, list(range(len(ids))))]).cpu()
        ref_runner.free_request(rid)
    del ref_runner
    torch.cuda.empty_cache()
    e32 = rel_err(torch.stack([ref[rid][p] for _, _, rid, p in sample]), torch.stack([plain[rid, p] for _, _, rid, p in sample]))
    assert e32 < FAMILY_TOL["float32"], e32
    pages = traces.peak_tokens(steps, round_to=16) // 16
    runner = load_runner(folder, torch.bfloat16, num_pages=pages, max_requests=4)
    got, want, at = {}, [], {}
    for st in steps:
        for e in st["entries"]:
            if not runner.has_request(e["id"]):
                runner.add_request(e["id"])
        logits = runner.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in st["entries"]])
        if st["step"] in expected:
            got[st["step"]] = logits.float().cpu()
            want += [ref[rid][p] for rid, p in expected[st["step"]]]
        for rid in st["end"]:
            runner.free_request(rid)
    e16 = rel_err(torch.stack([got[step][i] for step, i, _, _ in sample]), torch.stack([plain[rid, p] for _, _, rid, p in sample]))
    e = rel_err(torch.cat([got[k] for k in sorted(got)]), torch.stack(want))
    print(f"7B layer, mixed requests, seed {seed}: float32 {e32:.2e} and bfloat16 {e16:.2e} against the plain model on {len(sample)} rows; "
          f"bfloat16 against float32 {e:.2e} over {len(want)} rows, steps of {rows_per_step[0]}-{rows_per_step[-1]} rows", flush=True)
    assert e16 < DISTANCE_TOL_BF16 and e < FAMILY_TOL["bfloat16"]["7B"], (e16, e)
    runner.manager.check()
    assert runner.manager.free_pages() == [pages]
