"""Command line in the manner of the reference's inferctl (cli/main.cpp:553-556, 1601-1640:
``inferctl completion --prompt ... [--model M] [--max-tokens N] [--stream]``) and of its direct
engine probe (tests/tools/first_token_probe.cpp:38-126: --model, --prompt / --prompt-file,
--max-tokens, --ctx-size, --batch-size, --max-parallel-sequences; JSON on standard output).
The reference's inferctl talks to a server; this one drives the engine in the same process.

    inferctl completion --model DIR --prompt-ids 1,2,3 --max-tokens 16 [--stream]
    inferctl completion --random-weights config.json --seed 0 --prompt-ids 1,2,3
    inferctl random-weights --config config.json --out DIR --seed 0 [--shards N]
    inferctl inspect --model DIR
"""
from __future__ import annotations

import argparse
import json
import os
import sys
from typing import List, Optional


def _read_ids(args) -> List[List[int]]:
    prompts: List[List[int]] = []
    for s in args.prompt_ids or []:
        prompts.append([int(t) for t in s.replace(" ", "").split(",") if t])
    if args.prompt_ids_file:
        with open(args.prompt_ids_file) as f:
            for line in f:
                line = line.strip()
                if line:
                    prompts.append(json.loads(line) if line.startswith("[") else [int(t) for t in line.replace(",", " ").split()])
    texts = list(args.prompt or [])
    if args.prompt_file:
        with open(args.prompt_file) as f:
            texts.append(f.read())
    if texts:
        tok = _tokenizer(args.model)
        if tok is None:
            raise SystemExit(f"--prompt needs tokenizer.json in the model folder ({args.model}); pass token ids with --prompt-ids instead")
        prompts += [tok.encode(t).ids for t in texts]
    if not prompts:
        raise SystemExit("--prompt-ids, --prompt-ids-file or --prompt is required")
    return prompts


def _tokenizer(folder: Optional[str]):
    if not folder:
        return None
    path = os.path.join(folder, "tokenizer.json")
    if not os.path.isfile(path):
        return None
    from tokenizers import Tokenizer
    return Tokenizer.from_file(path)


def load_spec_from_args(args):
    """The ``ModelLoadSpec`` the options of ``completion`` describe (a complaint about them ends the program)."""
    from .engine.load_spec import LoadSpecError, ModelLoadSpec
    try:
        return ModelLoadSpec(path=args.model, random_weights=args.random_weights, seed=args.seed, dtype=args.dtype,
                             device=args.device, context_size=args.ctx_size, max_parallel_sequences=args.max_parallel_sequences,
                             kv_pages=args.kv_pages, page_size=args.page_size, max_batch_tokens=args.batch_size,
                             chunked_prefill_tokens=args.chunked_prefill_tokens, prefill_tokens_alone=args.prefill_tokens_alone,
                             decode_weight_copy=not args.no_decode_weight_copy,
                             strict_weights=not args.allow_unused_tensors, phase_timing=args.phase_timing,
                             library_gemm_tuning=args.gemm_tuning).checked()
    except LoadSpecError as e:
        raise SystemExit(f"inferctl: {e}")


def cmd_completion(args) -> int:
    from . import SamplingParams
    from .engine.engine import Engine, quiet_garbage_collector
    spec = load_spec_from_args(args)
    prompts = _read_ids(args)
    engine = Engine.load(spec)
    quiet_garbage_collector()
    params = SamplingParams(temperature=args.temperature, top_p=args.top_p, top_k=args.top_k, min_p=args.min_p,
                            frequency_penalty=args.frequency_penalty, presence_penalty=args.presence_penalty,
                            repetition_penalty=args.repetition_penalty, penalty_last_n=args.penalty_last_n,
                            seed=args.sample_seed if args.sample_seed is not None else 0xFFFFFFFF, max_tokens=args.max_tokens,
                            ignore_eos=args.ignore_eos, logprobs=args.top_n)
    tok = _tokenizer(args.model)

    def on_token(rid, t):
        if args.stream:
            print(json.dumps({"request": rid, "token": t, **({"text": tok.decode([t])} if tok else {})}), flush=True)

    outs = engine.generate(prompts, params, on_token)
    for o in outs:
        rec = {"model": args.model or args.random_weights, "request": o.request_id, "prompt_tokens": len(o.prompt_token_ids),
               "completion_tokens": len(o.token_ids), "token_ids": o.token_ids, "finish_reason": o.finish_reason}
        if o.logprobs is not None:
            rec["logprobs"] = [{"token": l.token_id, "logprob": round(l.logprob, 6),
                                "top_logprobs": [[t, round(v, 6)] for t, v in l.top_logprobs]} for l in o.logprobs]
        if tok:
            rec["completion"] = tok.decode(o.token_ids)
        print(json.dumps(rec), flush=True)
    st = engine.stats
    print(json.dumps({"perf": {"prefill_ms": round(st.prefill_ms, 3), "decode_ms": round(st.decode_ms, 3),
                               "prompt_tokens": st.prompt_tokens, "generated_tokens": st.generated_tokens}}), file=sys.stderr)
    return 0


def cmd_random_weights(args) -> int:
    import torch
    from .config import config_from_dict
    from .weights import write_random_model
    with open(args.config) as f:
        cfg = config_from_dict(json.load(f))
    write_random_model(args.out, cfg, args.seed, {"bfloat16": torch.bfloat16, "float32": torch.float32}[args.dtype],
                       shards=args.shards)
    print(json.dumps({"written": args.out, "seed": args.seed, "dtype": args.dtype, "shards": args.shards}))
    return 0


def cmd_inspect(args) -> int:
    from .config import load_config
    from .engine.model import Model
    from .weights import open_model_files
    cfg = load_config(args.model)
    specs = Model.param_specs_for(cfg)
    files = open_model_files(args.model)
    have = {n: (f.dtype(n), f.shape(n)) for f in files for n in f.names()}
    print(json.dumps({"config": cfg.to_dict(), "tensors_expected": len(specs), "tensors_in_file": len(have),
                      "missing": sorted(set(specs) - set(have)), "unexpected": sorted(set(have) - set(specs)),
                      "parameters": sum(int(__import__("math").prod(s)) for _, s in have.values())}, indent=2))
    return 0


def main(argv: Optional[List[str]] = None) -> int:
    ap = argparse.ArgumentParser(prog="inferctl", description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    sub = ap.add_subparsers(dest="command", required=True)
    c = sub.add_parser("completion", help="generate tokens for one or more prompts")
    c.add_argument("--model", help="folder with config.json and model.safetensors (or its shards and their index)")
    c.add_argument("--random-weights", metavar="CONFIG_JSON",
                   help="instead of --model: make seeded random weights for the model this config.json describes")
    c.add_argument("--seed", type=int, default=0, help="seed of --random-weights")
    c.add_argument("--prompt", action="append", help="text (needs tokenizer.json in the model folder)")
    c.add_argument("--prompt-file")
    c.add_argument("--prompt-ids", action="append", help="comma-separated token ids; may be given several times")
    c.add_argument("--prompt-ids-file", help="one prompt a line: a JSON list or ids separated by spaces/commas")
    c.add_argument("--max-tokens", "--max_tokens", type=int, default=16)
    c.add_argument("--stream", action="store_true", help="print each token as it is sampled")
    c.add_argument("--temperature", type=float, default=1.0, help="0 = greedy")
    c.add_argument("--top-p", type=float, default=1.0)
    c.add_argument("--top-k", type=int, default=0)
    c.add_argument("--min-p", type=float, default=0.0)
    c.add_argument("--frequency-penalty", type=float, default=0.0)
    c.add_argument("--presence-penalty", type=float, default=0.0)
    c.add_argument("--repetition-penalty", type=float, default=1.0)
    c.add_argument("--penalty-last-n", type=int, default=64)
    c.add_argument("--sample-seed", type=int, default=None, help="seed of the sampler's draws (default: a fresh one per request)")
    c.add_argument("--ignore-eos", action="store_true")
    c.add_argument("--top-n", type=int, default=None,
                   help="report each token's log-probability with the N most probable alternatives (0: the token's only)")
    c.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16")
    c.add_argument("--ctx-size", type=int, default=4096, help="tokens of context per sequence the cache is sized for")
    c.add_argument("--batch-size", type=int, default=16384, help="most tokens in one step (max_batch_tokens)")
    c.add_argument("--max-parallel-sequences", type=int, default=32, help="most requests in one step (max_batch_size)")
    c.add_argument("--chunked-prefill-tokens", type=int, default=512,
                   help="largest portion of a prompt in a step beside requests that are decoding")
    c.add_argument("--prefill-tokens-alone", type=int, default=None,
                   help="largest portion in a step in which nobody decodes (default: 2048, or --chunked-prefill-tokens if that is more)")
    c.add_argument("--kv-pages", type=int, default=None, help="pages in the cache (overrides --ctx-size)")
    c.add_argument("--page-size", type=int, default=16, help="tokens per page of the cache")
    c.add_argument("--device", default=None, help="rocm:N or cuda:N (the same ordinal); default: the current device")
    c.add_argument("--allow-unused-tensors", action="store_true",
                   help="tensors in the file that the model does not read are a warning instead of an error")
    c.add_argument("--no-decode-weight-copy", action="store_true",
                   help="keep one copy of the weights only (saves their size in memory, decoding is slower)")
    c.add_argument("--phase-timing", action="store_true",
                   help="print per-phase GPU times of every forward pass (decode steps then run kernel by kernel, not as graphs)")
    c.add_argument("--gemm-tuning", action="store_true",
                   help="let the library time its kernels for the matrix-product shapes of prompts (faster prompts once a shape "
                        "is known; the first product of a shape takes up to 0.3 s longer)")
    c.set_defaults(fn=cmd_completion)
    r = sub.add_parser("random-weights", help="write a model folder with seeded random weights")
    r.add_argument("--config", required=True, help="a config.json")
    r.add_argument("--out", required=True)
    r.add_argument("--seed", type=int, default=0)
    r.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16")
    r.add_argument("--shards", type=int, default=1, help="write this many safetensors files and an index")
    r.set_defaults(fn=cmd_random_weights)
    i = sub.add_parser("inspect", help="print a model folder's config and check its tensors against it")
    i.add_argument("--model", required=True)
    i.set_defaults(fn=cmd_inspect)
    args = ap.parse_args(argv)
    return args.fn(args)


if __name__ == "__main__":
    sys.exit(main())
