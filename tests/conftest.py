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
