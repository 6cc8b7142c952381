"""The typed load spec every entry point builds (no GPU): defaults, complaints in the reference's manner
(model/model_load_spec.cpp:38-59: the first thing wrong, as a sentence), and what the command line makes of its options."""
import pytest

from inferflux_amd.engine.load_spec import LoadSpecError, ModelLoadSpec


def test_defaults_are_the_references():
    s = ModelLoadSpec(path="m").checked()
    # scheduler/scheduler.h:64-89 (32 requests, 16384 tokens, portions of 512), native_bootstrap_config.h (pages of 16)
    assert (s.max_parallel_sequences, s.max_batch_tokens, s.chunked_prefill_tokens, s.page_size) == (32, 16384, 512, 16)
    assert s.dtype == "bfloat16" and s.kv_pages is None and s.cache_tokens == 4096 * 32 and s.strict_weights


@pytest.mark.parametrize("fields, complaint", [
    (dict(), "exactly one of path and random_weights"),
    (dict(path="m", random_weights="c.json"), "exactly one of path and random_weights"),
    (dict(path="m", dtype="fp8"), "dtype must be bfloat16 or float32"),
    (dict(path="m", device="gpu0"), "device must be cuda:N or rocm:N"),
    (dict(path="m", context_size=0), "context_size must be positive"),
    (dict(path="m", max_parallel_sequences=0), "max_parallel_sequences must be between 1 and 256"),
    (dict(path="m", max_parallel_sequences=257), "max_parallel_sequences must be between 1 and 256"),
    (dict(path="m", kv_pages=0), "kv_pages must be positive"),
    (dict(path="m", page_size=-16), "page_size must be positive"),
    (dict(path="m", max_batch_tokens=0), "max_batch_tokens must be positive"),
    (dict(path="m", chunked_prefill_tokens=0), "chunked_prefill_tokens must be positive"),
    (dict(random_weights="c.json", seed=-1), "seed must be nonnegative"),
])
def test_validate_names_the_first_problem(fields, complaint):
    s = ModelLoadSpec(**fields)
    assert complaint in s.validate()
    with pytest.raises(LoadSpecError, match=complaint):
        s.checked()


def test_from_mapping_and_devices():
    s = ModelLoadSpec.from_mapping({"path": "m", "context-size": 128, "max_parallel_sequences": 2, "device": "rocm:3", "kv_pages": None})
    assert (s.context_size, s.max_parallel_sequences, s.device_index, s.kv_pages) == (128, 2, 3, None)
    assert ModelLoadSpec(path="m", device="cuda:0").checked().device_index == 0
    assert ModelLoadSpec(path="m", dtype="fp32").checked().dtype == "fp32"
    with pytest.raises(LoadSpecError, match=r"unknown keys \['gpu_layers'\]"):
        ModelLoadSpec.from_mapping({"path": "m", "gpu_layers": 3})


def test_the_command_line_builds_the_spec_from_its_options():
    import argparse
    from inferflux_amd import cli
    captured = {}

    def fake_completion(args):
        captured["spec"] = cli.load_spec_from_args(args)
        return 0

    old = cli.cmd_completion
    cli.cmd_completion = fake_completion
    try:
        assert cli.main(["completion", "--random-weights", "cfg.json", "--seed", "5", "--prompt-ids", "1,2", "--page-size", "32",
                         "--kv-pages", "9", "--dtype", "float32", "--max-parallel-sequences", "3", "--batch-size", "77",
                         "--chunked-prefill-tokens", "11", "--ctx-size", "99", "--allow-unused-tensors"]) == 0
    finally:
        cli.cmd_completion = old
    s = captured["spec"]
    assert (s.path, s.random_weights, s.seed, s.page_size, s.kv_pages, s.dtype) == (None, "cfg.json", 5, 32, 9, "float32")
    assert (s.max_parallel_sequences, s.max_batch_tokens, s.chunked_prefill_tokens, s.context_size, s.strict_weights) == (3, 77, 11, 99, False)
    with pytest.raises(SystemExit, match="page_size must be positive"):
        cli.main(["completion", "--model", "m", "--prompt-ids", "1", "--page-size", "0"])
