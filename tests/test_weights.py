"""Weights: container, loading rule, the one error, random-weights folders (no GPU)."""
import json
import os
import struct

import pytest
import torch

from conftest import TINY, tiny_config
from inferflux_amd.engine.model import Model
from inferflux_amd.weights import (SafetensorsError, SafetensorsFile, WeightError, load_weights, storage_dtype,
                                   write_random_model, write_safetensors)


def test_container_roundtrip_against_the_safetensors_package(tmp_path):
    from safetensors.torch import load_file, save_file
    g = torch.Generator().manual_seed(0)
    tensors = {"a": torch.randn(3, 5, generator=g).bfloat16(), "b.c": torch.randn(7, generator=g),
               "i": torch.arange(6, dtype=torch.int32).view(2, 3), "h": torch.randn(2, 2, generator=g).half()}
    ours = str(tmp_path / "ours.safetensors")
    write_safetensors(ours, tensors, metadata={"format": "pt"})
    theirs = load_file(ours)                       # the independent reader accepts what we write
    for k, v in tensors.items():
        assert theirs[k].dtype == v.dtype and torch.equal(theirs[k], v)
    lib = str(tmp_path / "lib.safetensors")
    save_file(tensors, lib)
    f = SafetensorsFile(lib)                       # and we read what the independent writer writes
    assert sorted(f.names()) == sorted(tensors)
    for k, v in tensors.items():
        assert f.dtype(k) == v.dtype and torch.equal(f.tensor(k).clone(), v)
    f.close()


def test_truncated_and_malformed_files_name_the_problem(tmp_path):
    p = str(tmp_path / "t.safetensors")
    write_safetensors(p, {"w": torch.ones(64, 64)})
    blob = open(p, "rb").read()
    open(p, "wb").write(blob[:-100])
    with pytest.raises(SafetensorsError, match="'w'.*past the end"):
        SafetensorsFile(p)
    open(p, "wb").write(struct.pack("<Q", 1 << 40) + b"{}")
    with pytest.raises(SafetensorsError, match="header length"):
        SafetensorsFile(p)
    hdr = json.dumps({"w": {"dtype": "F32", "shape": [4], "data_offsets": [0, 8]}}).encode()
    open(p, "wb").write(struct.pack("<Q", len(hdr)) + hdr + b"\0" * 8)
    with pytest.raises(SafetensorsError, match="'w' holds 8 bytes"):
        SafetensorsFile(p)


def test_storage_rule():
    bf, f32, f16 = torch.bfloat16, torch.float32, torch.float16
    assert storage_dtype(bf, bf, False) == bf
    assert storage_dtype(f16, bf, False) == bf
    assert storage_dtype(f32, bf, False) == f32            # stored in 32-bit: stays so
    assert storage_dtype(bf, f32, False) == f32 and storage_dtype(f32, f32, False) == f32
    assert storage_dtype(torch.int64, bf, True) == torch.int32


def test_random_folder_loads_bit_equal_and_is_seeded(tmp_path, model_folders):
    from safetensors.torch import load_file
    for name, folder in model_folders.items():
        cfg = tiny_config(name)
        specs = Model.param_specs_for(cfg)
        raw = load_file(os.path.join(folder, "model.safetensors"))
        assert sorted(raw) == sorted(specs)
        for mode in (torch.bfloat16, torch.float32):
            got = load_weights(folder, specs, mode, "cpu")
            for n, t in got.items():
                assert t.dtype == mode and torch.equal(t.float(), raw[n].float()), n
        assert torch.equal(raw["model.norm.weight"].float(), torch.ones(cfg.hidden_size))
        w = raw["model.layers.0.mlp.gate_proj.weight"].float()
        assert abs(float(w.std()) - 0.02) < 0.002 and abs(float(w.mean())) < 0.002
    a, b, c = (str(tmp_path / x) for x in "abc")
    write_random_model(a, tiny_config("A"), seed=5)
    write_random_model(b, tiny_config("A"), seed=5)
    write_random_model(c, tiny_config("A"), seed=6)
    ta, tb, tc = (load_file(os.path.join(x, "model.safetensors")) for x in (a, b, c))
    assert all(torch.equal(ta[k], tb[k]) for k in ta)
    assert not torch.equal(ta["model.embed_tokens.weight"], tc["model.embed_tokens.weight"])


def test_a_tensor_stored_in_32_bit_stays_so(tmp_path):
    d = str(tmp_path / "m")
    cfg = tiny_config("A")
    write_random_model(d, cfg, seed=1, float32_tensors=("layernorm.weight", "model.norm.weight"))
    got = load_weights(d, Model.param_specs_for(cfg), torch.bfloat16, "cpu")
    assert got["model.norm.weight"].dtype == torch.float32
    assert got["model.layers.1.input_layernorm.weight"].dtype == torch.float32
    assert got["model.layers.1.mlp.up_proj.weight"].dtype == torch.bfloat16


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path, model_folders):
    from safetensors.torch import load_file
    cfg = tiny_config("B")
    raw = load_file(os.path.join(model_folders["B"], "model.safetensors"))
    del raw["model.layers.1.mlp.up_proj.weight"]
    del raw["model.norm.weight"]
    raw["model.layers.0.self_attn.q_norm.weight"] = torch.ones(24)
    raw["model.layers.2.self_attn.k_proj.weight"] = torch.zeros(48, 144)
    d = tmp_path / "broken"
    d.mkdir()
    cfg.save(str(d))
    write_safetensors(str(d / "model.safetensors"), raw)
    with pytest.raises(WeightError) as ei:
        load_weights(str(d), Model.param_specs_for(cfg), torch.bfloat16, "cpu")
    e = ei.value
    assert e.missing == ["model.layers.1.mlp.up_proj.weight", "model.norm.weight"]
    assert e.unexpected == ["model.layers.0.self_attn.q_norm.weight"]
    assert e.wrong_shape == [("model.layers.2.self_attn.k_proj.weight", (48, 144), (24, 144))]
    msg = str(e)
    assert "missing tensors (2)" in msg and "unexpected tensors (1)" in msg and "wrong shapes (1)" in msg


def test_config_and_file_are_cross_checked(tmp_path, model_folders):
    """A tied config with an lm_head in the file, or bias keys that disagree with the tensors, fail."""
    import shutil
    d = tmp_path / "x"
    shutil.copytree(model_folders["B"], d)
    cfg = json.load(open(d / "config.json"))
    cfg["tie_word_embeddings"] = True
    from inferflux_amd.config import config_from_dict
    with pytest.raises(WeightError) as ei:
        load_weights(str(d), Model.param_specs_for(config_from_dict(cfg)), torch.float32, "cpu")
    assert ei.value.unexpected == ["lm_head.weight"]
    cfg["tie_word_embeddings"] = False
    cfg["attention_bias"] = False
    with pytest.raises(WeightError) as ei:
        load_weights(str(d), Model.param_specs_for(config_from_dict(cfg)), torch.float32, "cpu")
    assert len(ei.value.unexpected) == 9 and all(n.endswith(".bias") for n in ei.value.unexpected)


def test_missing_files(tmp_path):
    with pytest.raises(WeightError, match="no safetensors files"):
        load_weights(str(tmp_path), {}, torch.float32, "cpu")


def test_shards_with_an_index_load_bit_equal(tmp_path, model_folders):
    """The layout of large checkpoints (the reference's rule: index's weight_map -> set of shard files,
    runtime/backends/cuda/inferflux_cuda_executor.cpp:366-402): same tensors, bit for bit, as one file."""
    cfg = tiny_config("B")
    specs = Model.param_specs_for(cfg)
    d = tmp_path / "sharded"
    write_random_model(str(d), cfg, seed=101, dtype=torch.bfloat16, shards=3)
    index = json.load(open(d / "model.safetensors.index.json"))
    shards = sorted(set(index["weight_map"].values()))
    assert len(shards) == 3 and all(os.path.isfile(d / s) for s in shards) and not os.path.exists(d / "model.safetensors")
    assert sorted(index["weight_map"]) == sorted(specs)
    sizes = [os.path.getsize(d / s) for s in shards]
    assert min(sizes) > 0.15 * sum(sizes)                               # dealt out by bytes, not all in one
    one = load_weights(model_folders["B"], specs, torch.bfloat16, "cpu")   # conftest wrote this one with the same seed
    many = load_weights(str(d), specs, torch.bfloat16, "cpu")
    assert sorted(one) == sorted(many) and all(torch.equal(one[k], many[k]) and one[k].dtype == many[k].dtype for k in one)
    # the independent reader sees the same tensors in the files the index names
    from safetensors.torch import load_file
    for s in shards:
        for k, v in load_file(str(d / s)).items():
            assert index["weight_map"][k] == s and torch.equal(v, one[k])


def test_broken_shard_sets_are_errors_that_name_the_file(tmp_path, model_folders):
    import shutil
    cfg = tiny_config("A")
    specs = Model.param_specs_for(cfg)
    d = tmp_path / "s"
    write_random_model(str(d), cfg, seed=1, shards=2)
    index_path = d / "model.safetensors.index.json"
    index = json.load(open(index_path))
    shards = sorted(set(index["weight_map"].values()))
    # a shard the index names is not there
    os.rename(d / shards[1], d / "elsewhere.safetensors")
    with pytest.raises(WeightError, match="shard files that do not exist.*" + shards[1].replace(".", r"\.")):
        load_weights(str(d), specs, torch.bfloat16, "cpu")
    os.rename(d / "elsewhere.safetensors", d / shards[1])
    # a tensor in two shards
    from safetensors.torch import load_file
    first = load_file(str(d / shards[0]))
    second = load_file(str(d / shards[1]))
    dup = next(iter(first))
    write_safetensors(str(d / shards[1]), {**second, dup: first[dup]})
    with pytest.raises(WeightError, match=f"'{dup}' appears in both"):
        load_weights(str(d), specs, torch.bfloat16, "cpu")
    write_safetensors(str(d / shards[1]), second)
    # shard names that leave the folder
    outside = tmp_path / "outside.safetensors"
    shutil.copy(d / shards[1], outside)
    for bad in ("../outside.safetensors", str(outside)):
        json.dump({"weight_map": {**index["weight_map"], dup: bad}}, open(index_path, "w"))
        with pytest.raises(WeightError, match="does not stay inside the model folder"):
            load_weights(str(d), specs, torch.bfloat16, "cpu")
    json.dump({"weight_map": {}}, open(index_path, "w"))
    with pytest.raises(WeightError, match="names no files"):
        load_weights(str(d), specs, torch.bfloat16, "cpu")
    json.dump(["not", "an", "index"], open(index_path, "w"))
    with pytest.raises(WeightError, match="not a safetensors index"):
        load_weights(str(d), specs, torch.bfloat16, "cpu")


def test_tensors_that_overlap_in_the_file_are_refused(tmp_path):
    p = str(tmp_path / "o.safetensors")
    hdr = json.dumps({"a": {"dtype": "F32", "shape": [4], "data_offsets": [0, 16]},
                      "b": {"dtype": "F32", "shape": [4], "data_offsets": [8, 24]}}).encode()
    open(p, "wb").write(struct.pack("<Q", len(hdr)) + hdr + b"\0" * 24)
    with pytest.raises(SafetensorsError, match="'a' and 'b' overlap"):
        SafetensorsFile(p)


def test_unused_tensors_are_an_error_or_a_reported_warning(tmp_path, model_folders, capfd):
    """Older exports carry buffers no part reads (rotary_emb.inv_freq): an error by default, a warning that lists
    them when the caller says so; what is missing or misshapen stays an error either way."""
    from safetensors.torch import load_file
    cfg = tiny_config("A")
    specs = Model.param_specs_for(cfg)
    raw = load_file(os.path.join(model_folders["A"], "model.safetensors"))
    raw["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.ones(8)
    d = tmp_path / "old"
    d.mkdir()
    cfg.save(str(d))
    write_safetensors(str(d / "model.safetensors"), raw)
    with pytest.raises(WeightError) as ei:
        load_weights(str(d), specs, torch.bfloat16, "cpu")
    assert ei.value.unexpected == ["model.layers.0.self_attn.rotary_emb.inv_freq"]
    report = {}
    got = load_weights(str(d), specs, torch.bfloat16, "cpu", strict=False, report=report)
    assert report["unused"] == ["model.layers.0.self_attn.rotary_emb.inv_freq"] and sorted(got) == sorted(specs)
    assert "1 tensors are not used by the model" in capfd.readouterr().err
    del raw["model.norm.weight"]
    write_safetensors(str(d / "model.safetensors"), raw)
    with pytest.raises(WeightError) as ei:
        load_weights(str(d), specs, torch.bfloat16, "cpu", strict=False)
    assert ei.value.missing == ["model.norm.weight"]
