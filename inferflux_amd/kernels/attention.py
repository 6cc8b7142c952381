"""Chooses the attention kernels for a step.

Every choice computes the same function (causal, optionally windowed, grouped-query attention
over the paged cache); they differ in speed and in which sizes they accept.  In bfloat16 with a
head size the matrix-core module takes, requests that bring at least TILE_MIN rows go to the
tile kernel (tiles of as many rows as the compiled module says; keys in splits when the tiles are
few and their pasts long) and all other rows (decode tokens, short portions) to the row kernel;
everything else (float32, other head sizes) goes to the plain kernel.
"""
from __future__ import annotations

from typing import Optional

import numpy as np
import torch

from . import ops

TILE_MIN = 16       # fewer rows than this are cheaper one by one
TILE_QT2_MIN_WORKGROUPS = 512   # two workgroups of the tile kernel for each of the 256 compute units
TILE_QT2_MIN_KEYS = 1536        # ... or rows that see this many keys on average, so that reading them from LDS half as often decides
TILE_SPLIT_BELOW = 384          # fewer workgroups than this: the tile kernel splits the keys
TILE_SPLIT_TARGET = 448         # ... aiming at this many workgroups,
TILE_SPLIT_MIN_KEYS = 512       # with at least this many keys to a split
TILE_SPLIT_MIN_LONGEST = 1536   # and only when the longest request has this many keys: writing and merging partial
                                # results costs about 20 us
TILE_SPLIT_FEW = 128            # at most this many workgroups: splits pay from
TILE_SPLIT_FEW_MIN_LONGEST = 1024   # this many keys on, and may be as short as
TILE_SPLIT_FEW_MIN_KEYS = 256       # this while the walk is short
TILE_MAX_SPLITS = 16
TILE_ORDER_MIN_ITEMS = 64       # launches of more workgroups than this get them in tile_order
ROW_CHUNK = 64      # keys per split of the row kernel: doubled while the launch keeps ROW_MIN_WAVES (ROW_MIN_WAVES_128
ROW_MIN_WAVES_128 = 1000   # for the step from 64 to 128) waves or more: a split costs a fixed start-up, so longer splits
ROW_MIN_WAVES = 1536       # pay when there are waves enough; and until a row has at most ROW_MAX_SPLITS splits.  The merge
ROW_MAX_SPLITS = 512       # launch shares a row of many splits among up to 8 waves, so one request over a long context may
                           # have hundreds (one row over 32,000 keys: 23.6 us in 250 splits against 35.8 in 125 with a
                           # merge of one wave; over 3,100 keys 11.8 us in 49 splits of 64 against 13.7 in 25 of 128).
ROW_WHOLE_MIN_PAIRS = 192   # (row, kv head) pairs from which a workgroup takes a pair's keys whole
ROW_WAVE_SLOTS = 2048       # waves the chip holds at the row kernel's two per SIMD


DIRECT_MIN_WORK = 1 << 18       # rows x keys seen per row from which the tall tiles of head size 128 win
DIRECT_SPLIT_FEW = 64           # at most this many workgroups: splits from 2,048 keys on,
DIRECT_SPLIT_BELOW = 128        # at most this many: from 3,072 keys on; more workgroups are never split
DIRECT_SPLIT_MIN_KEYS = 512


def _choose_direct(tiled_rows, tiled_keys, n_heads: int, rows_of, total: int, longest: int, seen: float):
    """``choose_tiling`` for head size 128, where the tall tiles are the kernel that loads straight into LDS.
    Measured (28, 16 and 40 query heads, workgroups in ``tile_order``; us with tiles of 64 / of 128 rows, each with
    its best number of splits): 512 rows 20 / 24, 1,024 rows 37 / 30, 2,048 rows 77 / 58, 8,192 rows 865 / 533;
    512 rows after 512 keys 34 / 27, after 3,584 keys 96 / 69 (85 whole), 1,024 after 3,072 141 / 93 (117 in two
    splits), 128 after 3,968 41 / 34 (83 whole), 2,048 after 6,144 436 / 226.  The tall tiles win wherever there
    is work enough, and their keys want cutting only for few workgroups with long walks."""
    n_big = sum(-(-int(n) // rows_of(2)) for n in tiled_rows)
    if total * seen < DIRECT_MIN_WORK or n_big * rows_of(2) > 2 * total:
        return None
    groups = n_big * n_heads
    splits, chunk = 1, 0
    if (groups <= DIRECT_SPLIT_FEW and longest >= 2048) or (groups <= DIRECT_SPLIT_BELOW and longest >= 3072):
        want = min(max(1, (2 * TILE_SPLIT_TARGET + groups) // (2 * groups)), longest // DIRECT_SPLIT_MIN_KEYS, TILE_MAX_SPLITS)
        if want > 1:
            chunk = (-(-longest // want) + 63) // 64 * 64
            splits = -(-longest // chunk)
            if splits <= 1:
                splits, chunk = 1, 0
    return 2, splits, chunk


def choose_tiling(tiled_rows, tiled_keys, n_heads: int, rows_of, tall_direct: bool = False):
    """(tiling: 1 = tiles of 64 rows, 2 = of 128; key splits; keys per split) for a launch of the tile kernel:
    ``tiled_rows`` the row counts of the requests it covers, ``tiled_keys`` how many keys each of them holds after
    the step, ``rows_of(qt)`` a tile's rows, ``tall_direct`` whether the tall tiles are the kernel of head size 128
    (``_choose_direct`` then decides whether to take them).  What follows is measured on the other kernel, whose
    tall tiles are two query tiles per wave.

    Measured at head size 128 (28, 16 and 40 query heads; portions of 256-8,192 rows after pasts of 0-7,680 keys,
    workgroups in ``tile_order``): two query tiles per wave win when they still give two workgroups to each compute
    unit (4,096 rows: 178 us against 236) or when a tile walks many keys on average (2,048 rows after 2,048 keys:
    158 us against 218; 1,024 after 1,024: 74 against 80), as long as the rows fill the taller tiles, and lose
    on a short causal prompt (2,048 rows: 81 us against 75).  About 448 workgroups are the best number to cut the
    keys for (1,024 rows after 7,168 keys: 292 us whole, 199 in two splits, 208 in four), and a cut pays only when
    the walk it shortens is long (512 rows after 512 keys: 34 us whole, 40 in two splits)."""
    total = int(sum(tiled_rows))
    longest = int(max(tiled_keys))
    # keys a row sees, averaged over the launch's rows: a request's rows see from (keys - rows) to keys of them
    seen = sum(int(n) * (int(k) - int(n) / 2.0) for n, k in zip(tiled_rows, tiled_keys)) / max(total, 1)
    n_big = sum(-(-int(n) // rows_of(2)) for n in tiled_rows)
    qt = 1
    if tall_direct:
        direct = _choose_direct(tiled_rows, tiled_keys, n_heads, rows_of, total, longest, seen)
        if direct is not None:
            return direct
    elif n_big * n_heads >= TILE_QT2_MIN_WORKGROUPS:
        qt = 2
    elif seen >= TILE_QT2_MIN_KEYS and n_big * rows_of(2) * 2 <= total * 3:
        qt = 2
    groups = sum(-(-int(n) // rows_of(qt)) for n in tiled_rows) * n_heads
    splits, chunk = 1, 0
    if groups < TILE_SPLIT_BELOW and longest >= (TILE_SPLIT_FEW_MIN_LONGEST if groups <= TILE_SPLIT_FEW else TILE_SPLIT_MIN_LONGEST):
        want = min(max(1, (2 * TILE_SPLIT_TARGET + groups) // (2 * groups)), longest // TILE_SPLIT_MIN_KEYS, TILE_MAX_SPLITS)
        if groups <= TILE_SPLIT_FEW and longest < 2 * TILE_SPLIT_MIN_LONGEST:
            want = max(want, min(4, longest // TILE_SPLIT_FEW_MIN_KEYS))
        if want > 1:
            chunk = (-(-longest // want) + 63) // 64 * 64
            splits = -(-longest // chunk)
            if splits <= 1:
                splits, chunk = 1, 0
    return qt, splits, chunk


from .device import CUS_PER_XCD, N_XCD      # the launch deals workgroups to the XCDs in turn, and an XCD its share to its compute units in turn


def tile_order(first_pos, last_pos, n_heads: int, window: Optional[int], splits: int, chunk: int, period: int = CUS_PER_XCD) -> np.ndarray:
    """Which work item each workgroup of a tile launch takes: int32 [8 * n], place x * n + i being the i-th workgroup
    of XCD x (-1: none).  ``first_pos`` / ``last_pos``: the positions of every tile's first and last row.

    A work item is (head, tile, split), numbered head * tiles * splits + (tiles - 1 - tile) * splits + split, and
    walks a number of 64-key tiles that is known here.  Workgroups on one compute unit share its time, so a unit
    that is given three long walks finishes long after one with three short ones: a causal prompt of 2,048 rows
    took 100 us in the order longest first, head by head, where the walks of the unit that came first summed to
    96 key tiles and the average was 58.  Here the items stay in head order (an XCD's workgroups read few kv heads,
    which its L2 then holds), are cut into eight runs of equal walks, not equal counts, and go to the workgroups
    of a run in boustrophedon order of their length with a compute unit's turn as the period, so that the i-th,
    (2 * period - 1 - i)-th, (2 * period + i)-th ... longest meet on one unit."""
    first_pos, last_pos = np.asarray(first_pos, np.int64), np.asarray(last_pos, np.int64)
    n_tiles = first_pos.shape[0]
    lo = np.maximum(first_pos - window + 1, 0) if window else np.zeros(n_tiles, np.int64)
    if splits > 1:
        s = np.arange(splits, dtype=np.int64)[None, :]
        lo_ts = np.maximum(lo[:, None], s * chunk)
        hi_ts = np.minimum(last_pos[:, None], (s + 1) * chunk - 1)
    else:
        lo_ts, hi_ts = lo[:, None], last_pos[:, None]
    walk = np.where(hi_ts >= lo_ts // 64 * 64, hi_ts // 64 - lo_ts // 64 + 1, 0)        # [tiles, splits] key tiles walked
    cost = (walk[::-1] + 1).reshape(-1)                                                # + 1: a workgroup's start and end
    cost = np.tile(cost, n_heads)                                                      # [items] in the kernel's numbering
    n_items = cost.shape[0]
    cum = np.cumsum(cost)
    run = np.minimum((cum - cost) * N_XCD // cum[-1], N_XCD - 1)                       # the run an item's start falls into
    counts = np.bincount(run, minlength=N_XCD)
    per_xcd = int(counts.max())
    order = np.full((N_XCD, per_xcd), -1, np.int32)
    start = 0
    for x in range(N_XCD):
        n = int(counts[x])
        if n == 0:
            continue
        items = np.arange(start, start + n)
        by_len = items[np.argsort(-cost[start:start + n], kind="stable")]
        rank = np.arange(n)
        row, col = rank // period, rank % period
        width = np.minimum(period, n - row * period)
        place = row * period + np.where(row % 2 == 0, col, width - 1 - col)
        order[x, place] = by_len
        start += n
    return order.reshape(-1)


def _work_lists(ctx, ctx_kv_heads, tile_rows, n_heads, tile_splits=1, tile_chunk=0, window=None, row_waves=8):
    """What the kernels need beyond the step's own arrays, computed once per step (and per number of
    kv heads, which decides how many waves a launch has)."""
    q_len, q_start, kv_len = ctx.h_q_len, ctx.h_q_start, ctx.h_kv_len
    tiled = q_len >= TILE_MIN
    tile_req, tile_q0 = [], []
    for r in np.nonzero(tiled)[0]:
        for q0 in range(0, int(q_len[r]), tile_rows):
            tile_req.append(r); tile_q0.append(q0)
    row_mask = ~tiled[ctx.h_row_req] if ctx.n_tokens else np.zeros(0, bool)
    rows = np.nonzero(row_mask)[0].astype(np.int32)
    out = {"n_tiles": len(tile_req), "n_rows": int(rows.size), "rows": None, "chunk": ROW_CHUNK, "max_splits": 1, "waves": 0,
           "tile_splits": 1, "tile_chunk": 0, "tile_row_list": None, "tile_order": None}
    lists = {}                       # everything that goes to the device, in one copy (each copy is a wait for the host)
    if tile_req:
        tile_req, tile_q0 = np.asarray(tile_req, np.int32), np.asarray(tile_q0, np.int32)
        lists["tile_req"], lists["tile_q0"] = tile_req, tile_q0
        if len(tile_req) * n_heads * tile_splits > TILE_ORDER_MIN_ITEMS:
            first = (kv_len[tile_req] - q_len[tile_req] + tile_q0).astype(np.int64)
            last = np.minimum(first + tile_rows, kv_len[tile_req]) - 1
            lists["tile_order"] = tile_order(first, last, n_heads, window, tile_splits, tile_chunk)
        # Few tiles with many keys each (portions of prompts with a long past) leave most of the chip idle
        # and each workgroup walking its keys alone: the keys are cut into splits that run side by side.
        if tile_splits > 1:
            out["tile_splits"], out["tile_chunk"] = tile_splits, tile_chunk
            lists["tile_row_list"] = np.nonzero(~row_mask)[0].astype(np.int32)
    if rows.size and rows.size != ctx.n_tokens:
        lists["rows"] = rows
    if lists:
        sizes = [(k, v.shape[0]) for k, v in lists.items()]
        packed = ctx.upload(np.concatenate([np.concatenate([v, np.zeros(-v.shape[0] % 4, np.int32)]) for v in lists.values()]))
        at = 0
        for k, n in sizes:
            out[k] = packed[at:at + n]
            at += n + -n % 4          # every list starts at a multiple of 16 bytes
    if rows.size:
        out["chunk"], out["waves"], out["max_splits"] = row_launch_shape(int(rows.size), ctx_kv_heads, ctx.kv_bound, row_waves)
    return out


def row_launch_shape(n_rows: int, n_kv_heads: int, max_kv: int, max_waves: int = 8):
    """(keys per split, waves per workgroup, splits) of a launch of the row kernel over ``n_rows`` rows whose requests
    hold at most ``max_kv`` keys (the bound of their block tables, not the lengths themselves: see
    StepContext.kv_bound).  ``max_waves``: what fits the kernel's LDS (``ops.row_waves_fit``).

    With (row, kv head) pairs enough to fill the chip by themselves, one workgroup takes a pair whole (keys per split
    0): its waves, as many as give the chip about one round of 2,048, share the row's keys evenly, meet in LDS and
    write the output, with no partial results in memory and no second launch.  Measured at 28 : 4 heads of 128 over
    3,100 keys, us whole / in splits with the merge launch: 48 rows 61 / 69, 64 rows 68 / 88, 96 rows 116 / 133, 128
    rows 129 / 178, 256 rows 250 / 361; 64 rows over 16,384 keys 328 / 358; 32 rows 57 / 48, so fewer pairs than 192
    keep the splits: their keys have to be spread over more compute units than there are pairs, which only a second
    launch can merge (one wave per split of ``chunk`` keys, waves per workgroup 0)."""
    pairs = n_rows * n_kv_heads
    if pairs >= ROW_WHOLE_MIN_PAIRS:
        waves = 1
        while waves * 2 <= min(max_waves, ROW_WAVE_SLOTS // pairs):
            waves *= 2
        return 0, waves, 1
    chunk = ROW_CHUNK
    while (-(-max_kv // chunk) > ROW_MAX_SPLITS
           or pairs * -(-max_kv // (2 * chunk)) >= (ROW_MIN_WAVES_128 if chunk == ROW_CHUNK else ROW_MIN_WAVES)):
        chunk *= 2
    return chunk, 0, -(-max_kv // chunk)


def paged_attention(q: torch.Tensor, cache, ctx, window: Optional[int], scale: float) -> torch.Tensor:
    """q [T, nH, d] of this step's rows against ``cache`` (a LayerCache); returns [T, nH*d]."""
    T, nH, d = q.shape
    table = ctx.block_table(cache.group)
    if not ops.mfma_attention_supported(q.dtype, d, cache.page_size) or cache.v.shape[2] != d:    # (values of another width: the plain kernel)
        return ops.attention_plain(q, cache.k, cache.v, ctx.row_req, ctx.positions, table, window, scale)
    n_kv = cache.k.shape[1]
    # Two query tiles per wave (128 rows per workgroup) read every key and value from LDS half as often.
    tiled = ctx.h_q_len >= TILE_MIN
    qt, splits, chunk = 1, 1, 0
    if tiled.any():
        qt, splits, chunk = choose_tiling(ctx.h_q_len[tiled], ctx.h_kv_len[tiled], nH, lambda t: ops.attention_tile_rows(d, t),
                                          tall_direct=d == ops.DIRECT_TILE_HEAD_DIM)
    tile_rows = ops.attention_tile_rows(d, qt)
    w = ctx.derived(("attention_work_lists", n_kv, tile_rows, nH, splits, chunk, window, d),
                    lambda: _work_lists(ctx, n_kv, tile_rows, nH, splits, chunk, window, ops.row_waves_fit(nH, n_kv, d, ops.ROW_MAX_WAVES)))
    out = torch.empty((T, nH * d), dtype=q.dtype, device=q.device)
    if w["n_tiles"]:
        ops.attention_tiles(q, cache.k, cache.v, out, w["tile_req"], w["tile_q0"], ctx.q_start, ctx.q_len, ctx.kv_len,
                            table, window, scale, qt, w["tile_chunk"], w["tile_splits"], w["tile_row_list"], ctx.row_req,
                            ctx.positions, w["tile_order"])
    if w["n_rows"]:
        ops.attention_rows(q, cache.k, cache.v, out, w["rows"], w["n_rows"], ctx.row_req, ctx.positions, table,
                           window, scale, w["chunk"], w["max_splits"], w["waves"], ctx.n_tokens == ctx.n_requests)
    return out
