"""Decode and prefill throughput of the engine at the Qwen2.5-7B shape, random weights, one GPU.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--layers L] [--batch B]

A step is one decode step of the whole engine (scheduler, step function, sampling); before the W warm-up steps of a
decode measurement its freshly captured graph is replayed SETTLE_STEPS times (see there; reported as ``settle_steps``).  Prints one
JSON line: decoded tokens a second at batch 8 as ``value``, the same at batch 1 and 64 under
``points`` (with their step times and roofline shares under ``ms_per_step_b1`` / ``roofline_b1`` and
``..._b64``), a 2,048-token prefill under ``prefill`` (the mean of ``mean_of`` runs with the library's
kernels chosen by timing, the best of them as ``best_ms``; ``prefill_untuned`` is the same with the library's
default choice, ``prefill_portions_512`` the same prompt in four portions of 512 tokens) and the
decode step's share of the HBM roofline under ``roofline``.  Every share is given against the data
sheet (``frac``) and, unless ``--no-ceilings``, against what this card gives a kernel that only reads
memory or a large library product (``frac_measured``, the ceilings under ``ceilings``).
"""
import argparse
import json
import sys
import time

HBM_GBS = 8000.0           # MI355X published HBM3E bandwidth, GB/s
PEAK_TFLOPS = {"bf16": 2500.0, "fp32": 157.3}

SHAPE_7B = dict(model_type="qwen2", architectures=["Qwen2ForCausalLM"], vocab_size=152064, hidden_size=3584,
                num_hidden_layers=28, num_attention_heads=28, num_key_value_heads=4, head_dim=128,
                intermediate_size=18944, max_position_embeddings=32768, rope_theta=1000000.0, rms_norm_eps=1e-6,
                tie_word_embeddings=False, attention_bias=True, use_sliding_window=False, torch_dtype="bfloat16")
# The two other workloads the family is sized for: many requests of mixed length with chunked
# prefill beside decoding (3B shape), and long prompts that stress cache capacity and long-context
# decode attention (14B shape).
SHAPE_3B = dict(SHAPE_7B, vocab_size=151936, hidden_size=2048, num_hidden_layers=36, num_attention_heads=16,
                num_key_value_heads=2, intermediate_size=11008, tie_word_embeddings=True)
SHAPE_14B = dict(SHAPE_7B, hidden_size=5120, num_hidden_layers=48, num_attention_heads=40, num_key_value_heads=8,
                 intermediate_size=13824, rms_norm_eps=1e-5)
# the family's small members: head size 64 and a hidden width of 7 x 128; twelve query heads on two kv heads
SHAPE_05B = dict(SHAPE_7B, vocab_size=151936, hidden_size=896, num_hidden_layers=24, num_attention_heads=14,
                 num_key_value_heads=2, head_dim=64, intermediate_size=4864, tie_word_embeddings=True)
SHAPE_15B = dict(SHAPE_7B, vocab_size=151936, hidden_size=1536, num_hidden_layers=28, num_attention_heads=12,
                 num_key_value_heads=2, intermediate_size=8960, tie_word_embeddings=True)
# the family's large members (the 72B shape's weights and their copy for small batches do not fit one card together:
# run it with --layers or --no-decode-weight-copy)
SHAPE_32B = dict(SHAPE_7B, hidden_size=5120, num_hidden_layers=64, num_attention_heads=40, num_key_value_heads=8,
                 intermediate_size=27648, rms_norm_eps=1e-5)
SHAPE_72B = dict(SHAPE_7B, hidden_size=8192, num_hidden_layers=80, num_attention_heads=64, num_key_value_heads=8,
                 intermediate_size=29568, rms_norm_eps=1e-5)
WORKLOADS = {
    "mixed3b": dict(shape=SHAPE_3B, name="Qwen2.5-3B shape", requests=64, prompt=(128, 2048), new=256, chunk=512),
    "long14b": dict(shape=SHAPE_14B, name="Qwen2.5-14B shape", requests=32, prompt=(8192, 8192), new=512, chunk=2048),
    # requests that finish one by one: the decode batch shrinks a request at a time, which is what captured decode
    # steps (one graph per layout) like least
    "staggered": dict(shape=SHAPE_7B, name="Qwen2.5-7B shape", requests=64, prompt=(512, 512), new=(32, 512), chunk=512),
}
CONTEXT = 4096
PROMPT = 2048
DECODE_KV_START = 3072      # mean context of a 2,048-token decode after a 2,048-token prompt
# Decode steps that every decode measurement runs, untimed, before its W warm-up steps.  A decode step is a replayed
# HIP graph, and the first replays of a graph that has just been captured run slower on this card (the 7B shape at
# batch 8: 3.44 ms for the first 37 replays, then 3.24 ms from one step to the next and for good, also after idling
# and for later requests on the same graph; 15 replays at batch 1; every weight-streaming kernel is 5-12 % slower in
# that phase, the same kernels on the same data).  An engine captures a layout once and replays it for as long as it
# serves, so the steady state is what a step costs; the contexts are counted as grown by these steps.
SETTLE_STEPS = 48
PAGE = 16


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--layers", type=int, default=None, help="run fewer layers than the shape has (both numbers are reported)")
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--dtype", choices=["bf16", "fp32"], default="bf16")
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 / 64 and prefill measurements")
    ap.add_argument("--no-gemm-tuning", action="store_true", help="leave the library's default kernel choice for large products")
    ap.add_argument("--workload", choices=["decode", "prefill", *WORKLOADS], default="decode",
                    help="decode: the headline measurement; prefill: only the 2,048-token prefill, --steps times "
                         "(for profiles); mixed3b / long14b: whole workloads through the scheduler")
    ap.add_argument("--no-decode-weight-copy", action="store_true",
                    help="decode from the weights' plain rows instead of the tiled copy")
    ap.add_argument("--ceilings", action=argparse.BooleanOptionalAction, default=True,
                    help="measure what the card gives (a 2 GB streaming read, an 8192^3 bf16 library product) once and "
                         "report every share against it beside the data sheet's peak")
    ap.add_argument("--context", type=int, default=DECODE_KV_START, help="tokens each request holds when the timed decode steps start")
    ap.add_argument("--shape", choices=["7b", "3b", "14b", "1.5b", "0.5b", "32b", "72b"], default="7b", help="layer sizes of the decode / prefill measurement (the headline is 7b)")
    ap.add_argument("--prompt-len", type=int, default=PROMPT, help="--workload prefill: tokens of the prompt")
    ap.add_argument("--prefill-chunk", type=int, default=0, help="--workload prefill: the prompt in portions of this many tokens, one step each (0: whole)")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        return 2
    kv_start = args.context

    import torch
    from inferflux_amd import SamplingParams
    from inferflux_amd.config import config_from_dict
    from inferflux_amd.engine.context import StepEntry
    from inferflux_amd.engine.engine import Engine
    from inferflux_amd.engine.model import Model
    from inferflux_amd.engine.runner import ModelRunner
    from inferflux_amd.engine.scheduler import SchedulerConfig

    from inferflux_amd.kernels import ops
    if not args.no_gemm_tuning:
        # Prefill and batch-64 products go to the library: let it time its kernels for the shapes that
        # are measured (not for the one-off shapes of the set-up).
        ops.enable_library_gemm_tuning(300)
        ops.pause_library_gemm_tuning(True)

    def note(msg):
        print(f"[bench] {msg}", file=sys.stderr, flush=True)
    ops.decode_weight_copy = not args.no_decode_weight_copy
    if args.workload in WORKLOADS:
        return run_workload(args, WORKLOADS[args.workload])
    shape = dict({"7b": SHAPE_7B, "3b": SHAPE_3B, "14b": SHAPE_14B, "1.5b": SHAPE_15B, "0.5b": SHAPE_05B, "32b": SHAPE_32B,
                  "72b": SHAPE_72B}[args.shape])
    shape_name = f"Qwen2.5-{args.shape.upper()} shape"
    layers_full = shape["num_hidden_layers"]
    if args.layers:
        shape["num_hidden_layers"] = args.layers
    cfg = config_from_dict(shape)
    tdt = {"bf16": torch.bfloat16, "fp32": torch.float32}[args.dtype]
    esz = 2 if args.dtype == "bf16" else 4
    dev = torch.device("cuda", 0)
    t0 = time.time()
    model = Model(cfg).init_random(0, tdt, dev)
    torch.cuda.synchronize()
    print(f"[bench] {cfg.num_hidden_layers}-layer model with random weights ready in {time.time() - t0:.1f} s", file=sys.stderr, flush=True)

    L, H, I, V = cfg.num_hidden_layers, cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size
    nH, nKV, d = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim
    layer_params = (nH + 2 * nKV) * d * H + (nH + 2 * nKV) * d + nH * d * H + 3 * I * H + 2 * H
    weight_bytes = (L * layer_params + H + V * H) * esz          # every weight a decode step uses, once (a tied head reads the table)
    kv_bytes_per_token = 2 * L * nKV * d * esz
    gen = torch.Generator().manual_seed(1)

    def make_engine(batch, kv_tokens):
        pages = batch * (-(-kv_tokens // PAGE) + 1)
        runner = ModelRunner(model, num_pages=pages, page_size=PAGE, max_requests=batch)
        return Engine(runner, SchedulerConfig(max_batch_size=batch, max_batch_tokens=16384, chunked_prefill_tokens=2048))

    def decode_rate(batch, steps, warmup):
        """tokens/s and ms/step of ``steps`` decode steps at ``batch`` with contexts from ``--context``."""
        # While the last prompts are still coming in, the first requests already decode: give every
        # request enough tokens (and pages) that none finishes before the timed steps are over.
        slack = -(-batch * kv_start // 16384) + 2 + SETTLE_STEPS
        eng = make_engine(batch, kv_start + steps + warmup + slack + 2)
        sp = SamplingParams(temperature=0.0, max_tokens=steps + warmup + slack + 1, ignore_eos=True)
        for _ in range(batch):
            eng.add_request(torch.randint(0, V, (kv_start,), generator=gen).tolist(), SamplingParams(**vars(sp)))
        while any(s.is_prefilling for s in eng.scheduler.running) or eng.scheduler.waiting:
            eng.step()                                            # prompts in; every request now decodes
        note(f"batch {batch}: prompts are in, decoding")
        ops.pause_library_gemm_tuning(False)
        for _ in range(SETTLE_STEPS + warmup):
            eng.step()
        ops.pause_library_gemm_tuning(True)
        torch.cuda.synchronize()
        t = time.perf_counter()
        for _ in range(steps):
            eng.step()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t
        assert len(eng.scheduler.running) == batch and eng.stats.preemptions == 0, "a request finished or was preempted while timing"
        kv_mean = kv_start + SETTLE_STEPS + warmup + steps / 2
        del eng
        torch.cuda.empty_cache()
        return batch * steps / dt, dt / steps * 1e3, kv_mean

    def prefill_rate(tokens, reps=3, chunk=0):
        """(tokens/s, ms, share of the matrix peak, best ms) of a prompt of ``tokens`` in one step (or in portions of
        ``chunk`` tokens, one step each): the mean of ``reps`` runs after one that warms up (and, with tuning on, lets
        the library time its kernels for these shapes), and the best of them beside it."""
        runner = ModelRunner(model, num_pages=-(-tokens // PAGE) + 1, page_size=PAGE, max_requests=2)
        ids = torch.randint(0, V, (tokens,), generator=gen).tolist()
        cuts = list(range(0, tokens, chunk or tokens))
        times = []
        ops.pause_library_gemm_tuning(False)
        for i in range(reps + 1):
            runner.add_request(i)
            torch.cuda.synchronize()
            t = time.perf_counter()
            for a0 in cuts:
                part = ids[a0:a0 + (chunk or tokens)]
                runner.step([StepEntry(i, part, [len(part) - 1] if a0 == cuts[-1] else [])])
            torch.cuda.synchronize()
            dt = time.perf_counter() - t
            runner.free_request(i)
            ops.pause_library_gemm_tuning(True)
            note(f"prefill of {tokens} tokens{f' in portions of {chunk}' if chunk else ''}: {dt * 1e3:.1f} ms")
            if i > 0:
                times.append(dt)
        mean = sum(times) / len(times)
        linear = 2.0 * tokens * L * ((nH + 2 * nKV) * d * H + nH * d * H + 3 * I * H) + 2.0 * V * H
        attn = 4.0 * L * nH * d * tokens * (tokens + 1) / 2
        return tokens / mean, mean * 1e3, (linear + attn) / mean / 1e12 / PEAK_TFLOPS[args.dtype], min(times) * 1e3

    def phase_shares(batch, steps=4):
        """Where the GPU's time goes, part by part: shares of the time between events recorded around each part in
        steps that are run kernel by kernel (not as a graph): a prompt of ``PROMPT`` tokens, then decode steps at
        ``batch`` with the contexts of the timed run.  Eager steps of few rows leave the GPU waiting for the host
        now and then, which is booked to the part that was being launched; the graphs' own times are the
        ``ms_per_step`` figures."""
        from inferflux_amd.engine.tracing import PhaseTimer
        runner = ModelRunner(model, num_pages=batch * (-(-(kv_start + steps) // PAGE) + 1), page_size=PAGE, max_requests=batch,
                             phase_timing=True)
        runner.timer.quiet = True
        out = {}
        for name, n_steps, tokens in ((f"prefill_{PROMPT}", 1, PROMPT), (f"decode_b{batch}", steps, 1)):
            if name.startswith("prefill"):
                runner.add_request("p")
                runner.step([StepEntry("p", torch.randint(0, V, (PROMPT,), generator=gen).tolist(), [PROMPT - 1])])   # warms the library up
                runner.free_request("p")
                runner.add_request("p")
                runner.timer = PhaseTimer(quiet=True)
                runner.step([StepEntry("p", torch.randint(0, V, (PROMPT,), generator=gen).tolist(), [PROMPT - 1])])
                runner.free_request("p")
            else:
                runner.timer = PhaseTimer(quiet=True)
                for r in range(batch):
                    runner.add_request(r)
                    for a0 in range(0, kv_start, 8192):
                        runner.step([StepEntry(r, torch.randint(0, V, (min(8192, kv_start - a0),), generator=gen).tolist(), [])])
                runner.step([StepEntry(r, [1], [0]) for r in range(batch)])
                runner.timer = PhaseTimer(quiet=True)
                for _ in range(n_steps):
                    runner.step([StepEntry(r, [1], [0]) for r in range(batch)])
            totals = dict(runner.timer.totals)
            total = sum(totals.values())
            out[name] = {k: round(v, 4) for k, v in runner.timer.shares().items()}
            out[name]["ms_eager"] = round(total / n_steps, 3)
            # what each stage moves or computes per step, over its time: GB/s of weights and cache for decoding (a stage is
            # bound by reading them once), TFLOP/s for the prompt
            if tokens == 1:
                kv = kv_start + 1 + n_steps / 2
                work = {"mixer.qkv": L * (nH + 2 * nKV) * d * (H + 1) * esz, "mixer.attention": L * batch * kv * 2 * nKV * d * esz,
                        "mixer": L * nH * d * H * esz, "ffn.gate_up": L * 2 * I * H * esz, "ffn": L * I * H * esz, "lm_head": V * H * esz}
                out[name + "_GBs"] = {k: round(b / (totals[k] / n_steps * 1e-3) / 1e9, 1) for k, b in work.items() if totals.get(k, 0) > 0}
            else:
                T = tokens
                work = {"mixer.qkv": 2.0 * T * L * (nH + 2 * nKV) * d * H, "mixer.attention": 4.0 * L * nH * d * T * (T + 1) / 2,
                        "mixer": 2.0 * T * L * nH * d * H, "ffn.gate_up": 2.0 * T * L * 2 * I * H, "ffn": 2.0 * T * L * I * H}
                out[name + "_TFLOPs"] = {k: round(f / (totals[k] * 1e-3) / 1e12, 1) for k, f in work.items() if totals.get(k, 0) > 0}
        out["how"] = ("events around each part of steps run kernel by kernel, waits for the host included: the GB/s and TFLOP/s here are "
                      "lower bounds of what the kernels reach inside a replayed step, whose own time is ms_per_step")
        del runner
        torch.cuda.empty_cache()
        return out

    def measured_ceilings():
        """What this card gives a kernel that only reads 2 GB (streaming loads), and the library's 8192^3 bfloat16
        product: the yardsticks beside the data sheet's 8 TB/s and 2.5 PFLOP/s."""
        from inferflux_amd.kernels.microbench import _time_us
        pool = torch.zeros((6 << 30) // 4, dtype=torch.float32, device=dev)
        n = (2 << 30) // 4
        t = min(_time_us(lambda i: ops.stream_read(pool[(i % 3) * n:(i % 3 + 1) * n], 2048, True), 6) for _ in range(2))
        read = (2 << 30) / t / 1e3                    # GB/s
        del pool
        a = torch.randn(8192, 8192, device=dev, dtype=torch.bfloat16)
        b = torch.randn(8192, 8192, device=dev, dtype=torch.bfloat16)
        t = min(_time_us(lambda i: torch.matmul(a, b.t()), 6) for _ in range(2))
        del a, b
        torch.cuda.empty_cache()
        return {"read_2GB_GBs": round(read, 1), "library_bf16_8192_TFLOPs": round(2 * 8192 ** 3 / t / 1e6, 1)}

    def hbm_roofline(batch, ms, kv_mean, ceil):
        step_bytes = weight_bytes + batch * kv_mean * kv_bytes_per_token
        achieved = step_bytes / (ms * 1e-3) / 1e9
        r = {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_GBS, "unit": "GB/s", "frac": round(achieved / HBM_GBS, 4)}
        if ceil:
            r["frac_measured"] = round(achieved / ceil["read_2GB_GBs"], 4)
        return r

    if args.workload == "prefill":
        ptps, pms, pfrac, _ = prefill_rate(args.prompt_len, reps=args.steps, chunk=args.prefill_chunk)
        print(json.dumps({"metric": f"prefill tok/s, {args.prompt_len} tokens (" + shape_name + f", {args.dtype}, random weights)",
                          "value": round(ptps, 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": 1,
                          "ms_per_step": round(pms, 3), "higher_is_better": True, "dtype": args.dtype,
                          "config": {"model": shape_name, "num_hidden_layers": layers_full, "layers_run": L,
                                     "prompt_len": args.prompt_len, "prefill_chunk": args.prefill_chunk or args.prompt_len,
                                     "library_gemm_tuning": not args.no_gemm_tuning},
                          "frac_of_peak": round(pfrac, 4)}), flush=True)
        return 0
    ceil = measured_ceilings() if (args.ceilings and args.dtype == "bf16") else None
    if ceil:
        note(f"this card: {ceil['read_2GB_GBs']:.0f} GB/s for a 2 GB read, {ceil['library_bf16_8192_TFLOPs']:.0f} TFLOP/s for the library's 8192^3 product")
    tps, ms, kv_mean = decode_rate(args.batch, args.steps, max(args.warmup, 1))
    note(f"batch {args.batch}: {tps:.0f} tokens/s")
    out = {
        "metric": f"decode tok/s at batch {args.batch} (" + shape_name + f", {args.dtype}, random weights)",
        "value": round(tps, 2), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "settle_steps": SETTLE_STEPS, "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": args.dtype, "data": "synthetic (uniform random token ids, seeded N(0,0.02) weights)",
        "config": {"model": shape_name, "global_batch": args.batch, "seq_len": max(CONTEXT, kv_start + SETTLE_STEPS + args.steps + args.warmup), "parallelism": "1 GPU",
                   "num_hidden_layers": layers_full, "layers_run": L, "hidden_size": H, "num_attention_heads": nH,
                   "num_key_value_heads": nKV, "head_dim": d, "intermediate_size": I, "vocab_size": V,
                   "prompt_len": PROMPT, "decode_kv_start": kv_start, "kv_page_size": PAGE,
                   "tie_word_embeddings": bool(shape["tie_word_embeddings"]), "library_gemm_tuning": not args.no_gemm_tuning,
                   "decode_weight_copy": not args.no_decode_weight_copy},
        "roofline": hbm_roofline(args.batch, ms, kv_mean, ceil),
    }
    if ceil:
        out["ceilings"] = ceil
    if not args.no_points:
        reps = 3
        ptps, pms, pfrac, pbest = prefill_rate(PROMPT, reps)
        out["prefill"] = {"value": round(ptps, 1), "tokens": PROMPT, "ms": round(pms, 3), "frac": round(pfrac, 4),
                          "mean_of": reps, "best_ms": round(pbest, 3), "library_gemm_tuning": not args.no_gemm_tuning}
        if ceil:
            out["prefill"]["frac_measured"] = round(pfrac * PEAK_TFLOPS[args.dtype] / ceil["library_bf16_8192_TFLOPs"], 4)
        if not args.no_gemm_tuning:
            # the same prefill with the library's own default choice of kernels (no timing of candidates, no file of
            # earlier choices): what a first call gets
            import torch.cuda.tunable as tunable
            tunable.enable(False)
            utps, ums, ufrac, ubest = prefill_rate(PROMPT, reps)
            tunable.enable(True)
            out["prefill_untuned"] = {"value": round(utps, 1), "tokens": PROMPT, "ms": round(ums, 3), "frac": round(ufrac, 4),
                                      "mean_of": reps, "best_ms": round(ubest, 3)}
        # the same prompt in portions of 512 tokens: what a prompt gets that arrives while others are decoding (a prompt
        # that arrives alone goes in portions of 2,048: the figure above)
        ctps, cms, cfrac, cbest = prefill_rate(PROMPT, reps, chunk=512)
        out["prefill_portions_512"] = {"value": round(ctps, 1), "tokens": PROMPT, "ms": round(cms, 3), "frac": round(cfrac, 4),
                                       "mean_of": reps, "best_ms": round(cbest, 3)}
        points = {}
        for b in (1, 64):
            btps, bms, bkv = decode_rate(b, min(args.steps, 32), min(args.warmup, 4))
            points[f"decode_b{b}"] = round(btps, 2)
            out[f"ms_per_step_b{b}"] = round(bms, 4)
            out[f"roofline_b{b}"] = hbm_roofline(b, bms, bkv, ceil)
        out["points"] = points
        out["phases"] = phase_shares(args.batch)
    print(json.dumps(out), flush=True)
    return 0


def run_workload(args, w) -> int:
    """A whole workload through the engine: every request added at once, chunked prefill mixed with
    decoding, greedy sampling.  A step here is one engine step; the value is generated tokens a second."""
    import torch
    from inferflux_amd import SamplingParams
    from inferflux_amd.config import config_from_dict
    from inferflux_amd.engine.engine import Engine, quiet_garbage_collector
    from inferflux_amd.engine.model import Model
    from inferflux_amd.engine.runner import ModelRunner
    from inferflux_amd.engine.scheduler import SchedulerConfig

    shape = dict(w["shape"])
    if args.layers:
        shape["num_hidden_layers"] = args.layers
    cfg = config_from_dict(shape)
    tdt = {"bf16": torch.bfloat16, "fp32": torch.float32}[args.dtype]
    model = Model(cfg).init_random(0, tdt, torch.device("cuda", 0))
    gen = torch.Generator().manual_seed(2)
    lo, hi = w["prompt"]
    lens = torch.randint(lo, hi + 1, (w["requests"],), generator=gen).tolist()
    prompts = [torch.randint(0, cfg.vocab_size, (n,), generator=gen).tolist() for n in lens]
    new_lo, new_hi = w["new"] if isinstance(w["new"], tuple) else (w["new"], w["new"])
    news = torch.randint(new_lo, new_hi + 1, (w["requests"],), generator=gen).tolist()
    pages = sum(-(-(n + m) // PAGE) + 1 for n, m in zip(lens, news))
    runner = ModelRunner(model, num_pages=pages, page_size=PAGE, max_requests=w["requests"])
    eng = Engine(runner, SchedulerConfig(max_batch_size=w["requests"], max_batch_tokens=16384, chunked_prefill_tokens=w["chunk"],
                                         prefill_tokens_alone=w["chunk"]))      # (the workloads name their portion: no longer ones while nobody decodes)
    first, t0 = {}, time.perf_counter()

    def on_token(rid, tok):
        if rid not in first:
            first[rid] = time.perf_counter() - t0

    sps = lambda: [SamplingParams(temperature=0.0, max_tokens=m, ignore_eos=True) for m in news]
    if args.warmup > 0:
        # One untimed pass of the same workload: the library loads a kernel the first time a shape asks
        # for it, which costs up to a second per shape and has nothing to do with the steady state.
        eng.generate(prompts, sps())
        eng.stats = type(eng.stats)()
        print(f"[bench] warm-up pass done ({runner.graph_captures} decode layouts captured)", file=sys.stderr, flush=True)
    captures_before, replays_before = runner.graph_captures, runner.graph_replays
    quiet_garbage_collector()               # as the command line does once its model is loaded
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    outs = eng.generate(prompts, sps(), on_token)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    n_gen = sum(len(o.token_ids) for o in outs)
    ttft = sorted(first.values())
    out = {
        "metric": f"generated tok/s, {w['requests']} requests, prompts {lo}-{hi}, {new_lo}-{new_hi} new tokens each ({w['name']}, {args.dtype}, random weights)",
        "value": round(n_gen / dt, 1), "unit": "tokens/s", "n_gpus": 1, "steps": eng.stats.steps,
        "warmup": 1 if args.warmup > 0 else 0,
        "ms_per_step": round(dt / eng.stats.steps * 1e3, 3), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": args.dtype, "data": "synthetic (uniform random token ids, seeded N(0,0.02) weights)",
        "config": {"model": w["name"], "global_batch": w["requests"], "seq_len": hi + new_hi, "parallelism": "1 GPU",
                   "num_hidden_layers": w["shape"]["num_hidden_layers"], "layers_run": cfg.num_hidden_layers,
                   "hidden_size": cfg.hidden_size, "num_attention_heads": cfg.num_attention_heads,
                   "num_key_value_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
                   "intermediate_size": cfg.intermediate_size, "vocab_size": cfg.vocab_size,
                   "prompt_tokens": sum(lens), "chunked_prefill_tokens": w["chunk"], "kv_page_size": PAGE, "kv_pages": pages},
        "total_s": round(dt, 2), "prompt_tok_per_s_overall": round(sum(lens) / dt, 1),
        "ttft_s": {"min": round(ttft[0], 3), "median": round(ttft[len(ttft) // 2], 3), "max": round(ttft[-1], 3)},
        "preemptions": eng.stats.preemptions,
        "decode_graphs": {"captured_in_timed_pass": runner.graph_captures - captures_before,
                          "captured_in_all": runner.graph_captures, "replays_in_timed_pass": runner.graph_replays - replays_before},
        "steps_by_tokens": {f"<={k}": n for k, n in sorted(eng.stats.step_tokens.items())},
    }
    print(json.dumps(out), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
