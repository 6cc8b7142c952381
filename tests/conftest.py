import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a GPU (run with -m gpu on an MI355X)")


# Three tiny configurations of the architecture that differ in every size and option.
TINY = {
    # 2 layers, H = nH*d, GQA 4:2, tied head, no window
    "A": dict(model_type="qwen2", architectures=["Qwen2ForCausalLM"], vocab_size=512, hidden_size=64,
              num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2, head_dim=16,
              intermediate_size=176, max_position_embeddings=256, rope_theta=10000.0, rms_norm_eps=1e-6,
              tie_word_embeddings=True, attention_bias=True, use_sliding_window=False, hidden_act="silu",
              torch_dtype="bfloat16"),
    # 3 layers, MQA 6:1, head_dim 24 (no multiple of 16), untied head
    "B": dict(model_type="qwen2", architectures=["Qwen2ForCausalLM"], vocab_size=1000, hidden_size=144,
              num_hidden_layers=3, num_attention_heads=6, num_key_value_heads=1, head_dim=24,
              intermediate_size=400, max_position_embeddings=512, rope_theta=1000000.0, rms_norm_eps=1e-5,
              tie_word_embeddings=False, attention_bias=True, use_sliding_window=False, hidden_act="silu",
              torch_dtype="bfloat16"),
    # 4 layers, nH*d != H, GQA 6:3, no bias, window of 24 on layers 1.. (two cache groups)
    "C": dict(model_type="qwen2", architectures=["Qwen2ForCausalLM"], vocab_size=777, hidden_size=96,
              num_hidden_layers=4, num_attention_heads=6, num_key_value_heads=3, head_dim=32,
              intermediate_size=208, max_position_embeddings=384, rope_theta=500000.0, rms_norm_eps=3e-6,
              tie_word_embeddings=False, attention_bias=False, use_sliding_window=True, sliding_window=24,
              max_window_layers=1, hidden_act="silu", torch_dtype="bfloat16"),
}


def tiny_config(name):
    from inferflux_amd.config import config_from_dict
    return config_from_dict(TINY[name])


@pytest.fixture(scope="session")
def model_folders(tmp_path_factory):
    """name -> folder with config.json and model.safetensors (bfloat16-representable random
    weights, so the engine's two modes and the plain implementation read the same numbers)."""
    from inferflux_amd.weights import write_random_model
    out = {}
    for i, name in enumerate(TINY):
        d = tmp_path_factory.mktemp(f"tiny{name}")
        write_random_model(str(d), tiny_config(name), seed=100 + i, dtype=torch.bfloat16)
        out[name] = str(d)
    return out


def has_gpu():
    return torch.cuda.is_available()


def sharpen(src_folder, dst_folder, seed, qk_gain=10.0):
    """Rewrite a random model so that faults show: attention that is peaked (larger q/k matrices), a
    feed-forward that matters (larger gate/up), norm weights and biases that are not 1 and 0-like.
    Values stay bfloat16-representable."""
    import shutil
    from safetensors.torch import load_file
    from inferflux_amd.weights import write_safetensors
    os.makedirs(dst_folder, exist_ok=True)
    shutil.copy(os.path.join(src_folder, "config.json"), os.path.join(dst_folder, "config.json"))
    t = load_file(os.path.join(src_folder, "model.safetensors"))
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, w in t.items():
        w = w.float()
        if name.endswith(("q_proj.weight", "k_proj.weight")):
            w = w * qk_gain
        elif name.endswith(("gate_proj.weight", "up_proj.weight")):
            w = w * 4.0
        elif name.endswith(("layernorm.weight", "norm.weight")):
            w = w + 0.2 * torch.randn(w.shape, generator=g)
        elif name.endswith(".bias"):
            w = w * 10.0
        out[name] = w.to(torch.bfloat16)
    write_safetensors(os.path.join(dst_folder, "model.safetensors"), out)


# How much larger than N(0, 0.02) the q/k matrices of the test models are.  10 makes attention so
# peaked that a float32 run shows any misplaced key; for bfloat16 runs 5 is used, because at 10 the
# rounding of scores to 8 mantissa bits alone moves logits by several percent (a plain model
# evaluated in bfloat16 is then off by 5-40 %, at 5 by 1-10 %; the engine stays below 2 %).
QK_GAIN = {"float32": 10.0, "bfloat16": 5.0}


class _Folders(dict):
    """name -> folder of the float32 test model; [(name, dtype)] picks the model for that dtype."""
    def __missing__(self, key):
        raise KeyError(key)


@pytest.fixture(scope="session")
def sharp_folders(model_folders, tmp_path_factory):
    out = _Folders()
    for i, (name, src) in enumerate(model_folders.items()):
        for dtype, gain in QK_GAIN.items():
            d = str(tmp_path_factory.mktemp(f"sharp{name}{dtype}"))
            sharpen(src, d, 200 + i, gain)
            out[name, dtype] = d
        out[name] = out[name, "float32"]
    return out


_PLAIN_CACHE = {}


def plain_logits(folder, ids):
    """Whole-sequence logits [S, V] of the plain implementation in float64 (cached per call)."""
    import plain_model as pm
    key = (folder, tuple(ids))
    if key not in _PLAIN_CACHE:
        if folder not in _PLAIN_CACHE:
            _PLAIN_CACHE[folder] = pm.load_folder(folder, torch.float64)
        cfg, W = _PLAIN_CACHE[folder]
        _PLAIN_CACHE[key] = pm.forward(cfg, W, list(ids))
    return _PLAIN_CACHE[key]


def seeded_ids(seed, n, vocab):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


# Logits are compared relative to the largest logit of the row set: a float32 engine differs from
# the float64 plain model by rounding that accumulates over a few hundred operations; a bfloat16
# engine rounds every activation to 8 bits of mantissa.  The bfloat16 bounds are per configuration: the
# largest error any test of that configuration shows (A 0.96 %, B 1.33 %, C 2.51 %: its window makes single
# scores count for more; other shapes up to 1.3 %) and half as much again.  INFERFLUX_REL_ERR_LOG (below)
# writes what a run shows.
REL_TOL = {"float32": 2e-5, "bfloat16": 2e-2}
BF16_TOL = {"A": 1.5e-2, "B": 2e-2, "C": 3.7e-2}


def tol(dtype, name=None):
    """The bound for logits of configuration ``name`` (a key of TINY, or None for any other shape) in ``dtype``."""
    if dtype == "bfloat16":
        return BF16_TOL.get(name, REL_TOL["bfloat16"])
    return REL_TOL[dtype]


_REL_ERRS = []      # (test id, error) of every comparison of a run, for the summary below


def rel_err(got, want):
    want = want.double()
    e = float((got.double() - want).abs().max() / want.abs().max())
    _REL_ERRS.append((os.environ.get("PYTEST_CURRENT_TEST", "?").split(" ")[0], e))
    return e


def pytest_sessionfinish(session, exitstatus):
    """With INFERFLUX_REL_ERR_LOG=path: the largest relative error each test saw, one line a test, into that file
    (what the tolerances above are set from)."""
    path = os.environ.get("INFERFLUX_REL_ERR_LOG")
    if not path or not _REL_ERRS:
        return
    worst = {}
    for test, e in _REL_ERRS:
        worst[test] = max(worst.get(test, 0.0), e)
    with open(path, "w") as f:
        for test, e in sorted(worst.items()):
            f.write(f"{e:.3e}  {test}\n")
