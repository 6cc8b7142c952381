"""Configuration and registry (no GPU)."""
import json

import pytest

from conftest import TINY
from inferflux_amd.config import (ConfigError, Qwen2Config, config_from_dict, load_config, plan_for,
                                  registered_architectures)
from inferflux_amd.engine.model import Model


def test_reads_every_key_and_roundtrips(tmp_path):
    for name, d in TINY.items():
        cfg = config_from_dict(d)
        assert isinstance(cfg, Qwen2Config)
        for k in ("vocab_size", "hidden_size", "num_hidden_layers", "num_attention_heads", "num_key_value_heads",
                  "head_dim", "intermediate_size", "max_position_embeddings", "rope_theta", "rms_norm_eps",
                  "tie_word_embeddings", "attention_bias"):
            assert getattr(cfg, k) == d[k], (name, k)
        cfg.save(str(tmp_path / name))
        assert load_config(str(tmp_path / name)) == cfg


def test_defaults_follow_the_reference():
    d = dict(TINY["A"])
    del d["head_dim"], d["num_key_value_heads"], d["rope_theta"], d["rms_norm_eps"]
    cfg = config_from_dict(d)
    assert cfg.head_dim == d["hidden_size"] // d["num_attention_heads"]  # executor.cpp:555-559
    assert cfg.num_key_value_heads == d["num_attention_heads"]
    assert cfg.rope_theta == 10000.0 and cfg.rms_norm_eps == 1e-6         # executor.cpp:571-573, executor.h:97


def test_lookup_by_model_type_then_architectures():
    d = dict(TINY["A"])
    del d["model_type"]
    assert isinstance(config_from_dict(d), Qwen2Config)
    d = dict(TINY["A"], model_type="QWEN2")
    d.pop("architectures")
    assert isinstance(config_from_dict(d), Qwen2Config)
    with pytest.raises(ConfigError, match="registered: .*qwen2"):
        config_from_dict(dict(TINY["A"], model_type="gpt_neox", architectures=["GPTNeoXForCausalLM"]))
    with pytest.raises(ConfigError, match="neither"):
        config_from_dict({k: v for k, v in TINY["A"].items() if k not in ("model_type", "architectures")})
    assert "qwen2" in registered_architectures() and "qwen2forcausallm" in registered_architectures()


@pytest.mark.parametrize("patch,match", [
    ({"hidden_size": None}, "hidden_size"),
    ({"vocab_size": "512"}, "vocab_size"),
    ({"num_key_value_heads": 3}, "multiple"),
    ({"head_dim": 15}, "even"),
    ({"hidden_act": "gelu"}, "hidden_act"),
    ({"rope_scaling": {"type": "yarn", "factor": 4.0}}, "rope_scaling"),
    ({"use_sliding_window": True}, "sliding_window"),
    ({"use_sliding_window": True, "sliding_window": 8, "max_window_layers": 9}, "max_window_layers"),
    ({"tie_word_embeddings": 1}, "true/false"),
    ({"num_hidden_layers": 0}, "positive"),
])
def test_bad_configs_are_errors(patch, match):
    with pytest.raises(ConfigError, match=match):
        config_from_dict(dict(TINY["A"], **patch))


def test_missing_config_json_is_an_error(tmp_path):
    with pytest.raises(ConfigError, match="config.json"):
        load_config(str(tmp_path))
    (tmp_path / "config.json").write_text("{not json")
    with pytest.raises(ConfigError, match="JSON"):
        load_config(str(tmp_path))


def test_plan_has_the_configs_sizes_layer_by_layer():
    cfg = config_from_dict(TINY["C"])
    plan = plan_for(cfg)
    assert len(plan.layers) == 4 and [e.layer for e in plan.schedule] == [0, 1, 2, 3]
    windows = [l.mixer.args["window"] for l in plan.layers]
    assert windows == [None, 24, 24, 24]
    assert all(l.mixer.args["n_heads"] == 6 and l.mixer.args["n_kv_heads"] == 3 and l.mixer.args["head_dim"] == 32
               for l in plan.layers)
    assert plan.layers[0].norm_in.args["eps"] == 3e-6 and plan.final_norm.args["eps"] == 3e-6
    assert plan.lm_head.args["tied_to"] is None
    assert plan_for(config_from_dict(TINY["A"])).lm_head.args["tied_to"] == "model.embed_tokens.weight"


def test_param_specs_have_the_reference_names_and_shapes():
    # names: runtime/backends/cuda/native/weight_map.cpp:21-58
    specs = Model.param_specs_for(config_from_dict(TINY["B"]))
    assert specs["model.embed_tokens.weight"].shape == (1000, 144)
    assert specs["lm_head.weight"].shape == (1000, 144)
    assert specs["model.norm.weight"].shape == (144,)
    p = "model.layers.2"
    assert specs[f"{p}.self_attn.q_proj.weight"].shape == (6 * 24, 144)
    assert specs[f"{p}.self_attn.k_proj.weight"].shape == (24, 144)
    assert specs[f"{p}.self_attn.v_proj.bias"].shape == (24,)
    assert specs[f"{p}.self_attn.o_proj.weight"].shape == (144, 6 * 24)
    assert specs[f"{p}.mlp.gate_proj.weight"].shape == (400, 144)
    assert specs[f"{p}.mlp.down_proj.weight"].shape == (144, 400)
    assert specs[f"{p}.input_layernorm.weight"].init == ("ones",)
    assert len(specs) == 3 + 3 * 12
    a = Model.param_specs_for(config_from_dict(TINY["A"]))
    assert "lm_head.weight" not in a                       # tied
    c = Model.param_specs_for(config_from_dict(TINY["C"]))
    assert not any(n.endswith(".bias") for n in c)         # attention_bias false
    assert c["model.layers.0.self_attn.o_proj.weight"].shape == (96, 192)   # [H, nH*d], nH*d != H
