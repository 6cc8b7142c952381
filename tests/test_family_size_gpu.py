"""The kernels at the sizes of the model family (Qwen2.5-7B layer shape: hidden 3584, 28 query heads
on 4 kv heads of 128, feed-forward 18944, vocabulary 152064; two layers to keep it short): the
bfloat16 engine against the float32 engine on the same weights, under several cuttings.  The
float32 engine is the reference here; the tiny configurations tie it to the plain implementation."""
import pytest
import torch

from conftest import REL_TOL, rel_err, seeded_ids

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
        assert e < REL_TOL["bfloat16"], e
    assert all(r.manager.free_pages() == [96] for r in runners.values())
