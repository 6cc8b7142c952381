"""Timings of single kernels at chosen sizes, for profiles and for tuning launch shapes.

    python -m inferflux_amd.kernels.microbench attention-tiles --rows 8192 [--query-tiles 2]
    python -m inferflux_amd.kernels.microbench attention-rows --batch 64 --context 3072 [--chunk 512]
    python -m inferflux_amd.kernels.microbench gemm --rows 8 [--shape gate_up]
    python -m inferflux_amd.kernels.microbench sampling --batch 8 [--vocab 152064]
    python -m inferflux_amd.kernels.microbench ceilings

Sizes default to the Qwen2.5-7B shape (28 query heads, 4 kv heads, head size 128, hidden 3584,
intermediate 18944).  Times are averages of back-to-back launches between two events and include what
the Python wrapper costs per call (10-15 us): for kernels that short, read the kernel's own time from
``rocprofv3 --kernel-trace`` around this program instead.  Products rotate through enough copies of the
weight, and row attention through enough caches, that no launch finds its operands in a cache.
"""
from __future__ import annotations

import argparse
import math
import sys

import numpy as np
import torch

from . import ops

GEMM_SHAPES = {"qkv": (4608, 3584), "o": (3584, 3584), "gate_up": (37888, 3584), "down": (3584, 18944),
               "lm_head": (152064, 3584)}


def _time_us(fn, iters: int, graph: bool = False) -> float:
    """Average time of a call, after about 50 ms of the same calls (the card's clocks take that long to settle: a
    kernel of 0.5 ms timed after three warm-up calls reads 10-20 % slow).  ``graph``: the ``iters`` calls are captured
    as one HIP graph and the graph is replayed, so that kernels shorter than the host's 10-15 us per call are timed as
    they run inside a captured decode step, one behind the other."""
    import time
    if graph:
        fn(0)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for i in range(iters):
                fn(i)
        t0 = time.perf_counter()
        while time.perf_counter() - t0 < 0.05:
            g.replay()
            torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(5):
            g.replay()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) / (5 * iters) * 1e3
    t0 = time.perf_counter()
    n = 0
    while n < 3 or (time.perf_counter() - t0 < 0.05 and n < 2000):
        fn(n)
        n += 1
        if n % 8 == 0:
            torch.cuda.synchronize()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for i in range(iters):
        fn(i + 3)
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / iters * 1e3


def attention_tiles(args) -> None:
    dev, T, nH, nKV, d, P = "cuda", args.rows, args.heads, args.kv_heads, args.head_dim, args.page_size
    past = args.past
    L = past + T
    q = torch.randn(T, nH, d, device=dev, dtype=torch.bfloat16)
    nb = -(-L // P)
    kc = torch.randn(nb, nKV, P, d, device=dev, dtype=torch.bfloat16)
    vc = torch.randn(nb, nKV, d, P, device=dev, dtype=torch.bfloat16)
    table = torch.arange(nb, dtype=torch.int32, device=dev).view(1, nb)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=dev)
    row_req, positions = i32([0] * T), torch.arange(past, L, dtype=torch.int32, device=dev)
    row_list = torch.arange(T, dtype=torch.int32, device=dev)
    flops = 4.0 * nH * d * (T * past + T * (T + 1) / 2)
    for qt in ([args.query_tiles] if args.query_tiles else list(ops.TILE_QTS)):
        tiles = list(range(0, T, ops.attention_tile_rows(d, qt)))
        out = torch.empty(T, nH * d, device=dev, dtype=torch.bfloat16)
        for chunk in ([int(c) for c in args.tile_chunk.split(",")] if args.tile_chunk else [0]):
            splits = -(-L // chunk) if chunk else 1
            for period in [int(c) for c in args.order_period.split(",")]:
                order = None
                if period:
                    from .attention import tile_order
                    first = past + np.asarray(tiles)
                    order = torch.from_numpy(tile_order(first, np.minimum(first + ops.attention_tile_rows(d, qt), L) - 1, nH, None, splits,
                                                        chunk, period)).to(dev)
                call = (q, kc, vc, out, i32([0] * len(tiles)), i32(tiles), i32([0]), i32([T]), i32([L]), table, None, 1 / math.sqrt(d), qt,
                        chunk, splits, row_list if splits > 1 else None, row_req, positions, order)
                t = _time_us(lambda i: ops.attention_tiles(*call), args.iters)
                print(f"attention-tiles rows={T} past={past} query_tiles={qt} key splits={splits} order period={period}: {t:9.1f} us  "
                      f"{flops / t / 1e6:7.1f} TFLOP/s (visible keys only)", flush=True)


def attention_rows(args) -> None:
    dev, B, kv, nH, nKV, d, P = "cuda", args.batch, args.context, args.heads, args.kv_heads, args.head_dim, args.page_size
    nb = -(-kv // P)
    # enough caches to rotate through that no launch finds its keys and values in the last-level cache
    copies = max(2, int(args.rotate_gb * 1e9 // (2 * B * nb * nKV * P * d * 2)))
    k0 = torch.randn(B * nb, nKV, P, d, device=dev, dtype=torch.bfloat16)
    v0 = torch.randn(B * nb, nKV, d, P, device=dev, dtype=torch.bfloat16)
    caches = [(k0, v0)] + [(k0.clone(), v0.clone()) for _ in range(copies - 1)]
    # where a request's pages lie: anywhere, or one after the other as a pool hands them to a prompt that comes in whole
    order = torch.arange(B * nb, device=dev) if args.pages == "in-order" else torch.randperm(B * nb, device=dev)
    table = order.to(torch.int32).view(B, nb).contiguous()
    q = torch.randn(B, nH, d, device=dev, dtype=torch.bfloat16)
    out = torch.empty(B, nH * d, device=dev, dtype=torch.bfloat16)
    row_req = torch.arange(B, dtype=torch.int32, device=dev)
    pos = torch.full((B,), kv - 1, dtype=torch.int32, device=dev)
    bound = -(-kv // (64 * P)) * 64 * P if args.graph_width else kv   # a captured step's grid covers its block-table width
    gb = B * kv * nKV * d * 2 * 2 / 1e9
    for chunk in ([int(c) for c in args.chunk.split(",")] if args.chunk else [128, 256, 512, 1024]):
        splits = -(-bound // chunk)
        t = _time_us(lambda i: ops.attention_rows(q, *caches[i % copies], out, None, B, row_req, pos, table, None,
                                                  1 / math.sqrt(d), chunk, splits), args.iters, args.graph)
        print(f"attention-rows batch={B} context={kv} one wave per split of {chunk} keys ({splits} splits) + merge launch: "
              f"{t:8.1f} us  {gb / t * 1e3:5.2f} TB/s of cache", flush=True)
    for waves in [int(w) for w in args.waves.split(",") if w]:
        waves = ops.row_waves_fit(nH, nKV, d, waves)
        t = _time_us(lambda i: ops.attention_rows(q, *caches[i % copies], out, None, B, row_req, pos, table, None,
                                                  1 / math.sqrt(d), 0, 1, waves), args.iters, args.graph)
        print(f"attention-rows batch={B} context={kv} one workgroup of {waves} waves per (row, kv head): "
              f"{t:8.1f} us  {gb / t * 1e3:5.2f} TB/s of cache", flush=True)


def gemm(args) -> None:
    dev, M = "cuda", args.rows
    for name in ([args.shape] if args.shape else list(GEMM_SHAPES)):
        N, K = GEMM_SHAPES[name]
        copies = max(2, min(24, int(3e9 // (N * K * 2))))
        ws = [ops.prepare_linear(torch.randn(N, K, device=dev, dtype=torch.bfloat16)) for _ in range(copies)]
        x = torch.randn(M, K, device=dev, dtype=torch.bfloat16)
        gb = N * K * 2 / 1e9
        t = _time_us(lambda i: ops.linear(x, ws[i % copies]), args.iters, args.graph)
        t_lib = _time_us(lambda i: torch.matmul(x, ws[i % copies].rows.t()), args.iters, args.graph)
        print(f"gemm {name:8s} rows={M:3d} [{N} x {K}]: engine's choice {t:8.1f} us ({gb / t * 1e3:5.2f} TB/s of weights)   "
              f"library {t_lib:8.1f} us", flush=True)
        del ws


def sampling(args) -> None:
    """The sampling kernels on ``--batch`` rows of ``--vocab`` logits (a normal spread of ``--spread``), each call
    inside a replayed graph: greedy, a draw at a temperature, with top-k and top-p, with top-p alone (more
    candidates), and the log-probabilities with five alternatives."""
    dev, R, V = "cuda", args.batch, args.vocab
    logits = torch.randn(R, V, device=dev) * args.spread
    full = lambda v, dt=torch.float32: torch.full((R,), v, dtype=dt, device=dev)
    u = torch.rand(R, device=dev)
    chosen = ops.argmax(logits)
    t08, t1, k0, k50, p1, p09, m0, m001 = (full(0.8), full(1.0), full(0, torch.int32), full(50, torch.int32), full(1.0), full(0.9),
                                           full(0.0), full(0.01))
    cases = [("argmax", lambda i: ops.argmax(logits)),
             ("temperature 0.8", lambda i: ops.sample(logits, t08, k0, p1, m0, u, any_greedy=False, any_filters=False)),
             ("temperature 0.8, top-k 50, top-p 0.9", lambda i: ops.sample(logits, t08, k50, p09, m0, u, any_greedy=False)),
             ("temperature 0.8, top-p 0.9", lambda i: ops.sample(logits, t08, k0, p09, m0, u, any_greedy=False)),
             ("temperature 1, min-p 0.01", lambda i: ops.sample(logits, t1, k0, p1, m001, u, any_greedy=False, any_filters=False)),
             ("log-probabilities, 5 alternatives", lambda i: ops.logprobs(logits, chosen, 5)),
             ("log-probability of the token alone", lambda i: ops.logprobs(logits, chosen, 0))]
    for name, fn in cases:
        print(f"sampling rows={R} vocabulary={V} {name}: {_time_us(fn, args.iters, True):8.1f} us", flush=True)


def ceilings(args) -> None:
    """What a kernel that only reads (or copies) gets from this card's memory, and the library's large products."""
    dev = "cuda"
    pool = torch.zeros(int(args.pool_gb * 2**30) // 4, dtype=torch.float32, device=dev)
    pool_bytes = pool.numel() * 4
    for mb in (32, 128, 512, 2048):
        n = mb * 2**20 // 4
        if 2 * n > pool.numel():
            continue
        places = pool_bytes // (n * 4)            # each launch reads another piece of the pool: nothing is found in a cache
        for streaming in (False, True):
            best = None
            for waves in (2048, 4096, 8192):
                t = _time_us(lambda i: ops.stream_read(pool[(i % places) * n:(i % places + 1) * n], waves, streaming), args.iters)
                if best is None or t < best[0]:
                    best = (t, waves)
            print(f"read  {mb:5d} MB {'streaming' if streaming else 'plain    '} loads: {best[0]:8.1f} us  "
                  f"{mb * 2**20 / best[0] / 1e6:5.2f} TB/s  ({best[1]} waves)", flush=True)
    for mb in (128, 1024):
        n = mb * 2**20 // 4
        places = pool_bytes // (2 * n * 4)
        if places < 1:
            continue
        for streaming in (False, True):
            def copy(i):
                at = (i % places) * 2 * n
                ops.stream_copy(pool[at:at + n], pool[at + n:at + 2 * n], 4096, streaming)
            t = _time_us(copy, args.iters)
            print(f"copy  {mb:5d} MB {'streaming' if streaming else 'plain    '}: {t:8.1f} us  "
                  f"{2 * mb * 2**20 / t / 1e6:5.2f} TB/s read + written", flush=True)
    del pool
    for dtype, size in ((torch.bfloat16, 8192), (torch.float32, 4096)):
        a = torch.randn(size, size, device=dev, dtype=dtype)
        b = torch.randn(size, size, device=dev, dtype=dtype)
        t = _time_us(lambda i: torch.matmul(a, b.t()), args.iters)
        print(f"library product {size}^3 {str(dtype).split('.')[1]}: {t:8.1f} us  {2 * size**3 / t / 1e6:7.1f} TFLOP/s", flush=True)


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="python -m inferflux_amd.kernels.microbench")
    sub = ap.add_subparsers(dest="what", required=True)
    for name, fn in (("attention-tiles", attention_tiles), ("attention-rows", attention_rows), ("gemm", gemm),
                     ("sampling", sampling), ("ceilings", ceilings)):
        p = sub.add_parser(name)
        p.set_defaults(fn=fn)
        p.add_argument("--iters", type=int, default=10)
        if name in ("attention-rows", "gemm"):
            p.add_argument("--graph", action="store_true", help="time the calls inside a replayed HIP graph (kernels shorter than "
                           "the host's time per call)")
        if name.startswith("attention"):
            p.add_argument("--heads", type=int, default=28)
            p.add_argument("--kv-heads", type=int, default=4)
            p.add_argument("--head-dim", type=int, default=128)
            p.add_argument("--page-size", type=int, default=16)
        if name == "attention-tiles":
            p.add_argument("--rows", type=int, default=2048, help="rows of one request in one step, no past")
            p.add_argument("--query-tiles", type=int, default=0, help="1 or 2 query tiles per wave (0: both)")
            p.add_argument("--past", type=int, default=0, help="keys the request already holds (a later portion of a prompt)")
            p.add_argument("--order-period", default="0,32", help="workgroups ordered by attention.tile_order with these periods, "
                           "comma separated (0: in the order of the heads, longest first)")
            p.add_argument("--tile-chunk", default="", help="keys per split, comma separated (multiples of 64; empty or 0: no splits)")
        if name == "attention-rows":
            p.add_argument("--batch", type=int, default=8)
            p.add_argument("--context", type=int, default=3072)
            p.add_argument("--chunk", default="", help="keys per split, comma separated (empty: 128, 256, 512 and 1024)")
            p.add_argument("--waves", default="4,8", help="also: one workgroup of this many waves per (row, kv head), comma separated")
            p.add_argument("--graph-width", action="store_true", help="size the grid by the block-table width a captured step has "
                           "(the next multiple of 64 pages), not by the context")
            p.add_argument("--rotate-gb", type=float, default=2.0,
                           help="memory the launches rotate through (a model's step touches tens of GB between two uses of a cache)")
            p.add_argument("--pages", choices=["shuffled", "in-order"], default="shuffled", help="how a request's pages lie in the pool")
        if name == "sampling":
            p.add_argument("--batch", type=int, default=8)
            p.add_argument("--vocab", type=int, default=152064)
            p.add_argument("--spread", type=float, default=3.0, help="standard deviation of the logits")
        if name == "ceilings":
            p.add_argument("--pool-gb", type=float, default=16.0, help="memory the reads and copies rotate through")
        if name == "gemm":
            p.add_argument("--rows", type=int, default=8, help="rows of x")
            p.add_argument("--shape", choices=list(GEMM_SHAPES), default=None)
    args = ap.parse_args(argv)
    if not torch.cuda.is_available():
        print("microbench: no GPU", file=sys.stderr)
        return 2
    args.fn(args)
    return 0


if __name__ == "__main__":
    sys.exit(main())
