"""Builders of replay traces for the tests, in trace_run's JSON format, and the comparison of
what a replay wrote with whole-sequence logits.

A trace is a list of steps {"step", "entries": [{"id", "tokens", "want"}], "end"}.  ``expected``
maps a step number to the list of (request, position) whose logits that step writes, in order.
"""
import random


def whole(seqs):
    """Each request alone and whole: one step per request, every position wanted."""
    steps, expected = [], {}
    for i, (rid, ids) in enumerate(seqs.items()):
        steps.append({"step": i, "entries": [{"id": rid, "tokens": ids, "want": list(range(len(ids)))}], "end": [rid]})
        expected[i] = [(rid, p) for p in range(len(ids))]
    return steps, expected


def prefill_then_decode(seqs, tail=32):
    """Most of it in one step, the last ``tail`` tokens one by one (each request alone)."""
    steps, expected, n = [], {}, 0
    for rid, ids in seqs.items():
        head = max(1, len(ids) - tail)
        steps.append({"step": n, "entries": [{"id": rid, "tokens": ids[:head], "want": [head - 1]}], "end": []})
        expected[n] = [(rid, head - 1)]
        n += 1
        for p in range(head, len(ids)):
            steps.append({"step": n, "entries": [{"id": rid, "tokens": [ids[p]], "want": [0]}],
                          "end": [rid] if p == len(ids) - 1 else []})
            expected[n] = [(rid, p)]
            n += 1
        if head == len(ids):
            steps[-1]["end"] = [rid]
    return steps, expected


def portions(seqs, sizes=(5, 2, 11, 3, 2, 16, 1, 17, 2, 31, 4)):
    """Portions of changing size, down to two tokens and single ones, every position wanted."""
    steps, expected, n = [], {}, 0
    for rid, ids in seqs.items():
        p, k = 0, 0
        while p < len(ids):
            m = min(sizes[k % len(sizes)], len(ids) - p)
            steps.append({"step": n, "entries": [{"id": rid, "tokens": ids[p:p + m], "want": list(range(m))}],
                          "end": [rid] if p + m == len(ids) else []})
            expected[n] = [(rid, q) for q in range(p, p + m)]
            p += m; k += 1; n += 1
    return steps, expected


def mixed(seqs, seed=0, max_live=4, chunk_sizes=(2, 3, 7, 16, 24)):
    """Up to ``max_live`` requests at a time: portions of some beside single tokens of others, some
    left out of a step, requests ending while others go on and new ones taking their pages."""
    rng = random.Random(seed)
    waiting = list(seqs.items())
    live = {}            # rid -> [ids, next position, decode_from]
    steps, expected, n = [], {}, 0
    while waiting or live:
        while waiting and len(live) < max_live and (not live or rng.random() < 0.6):
            rid, ids = waiting.pop(0)
            live[rid] = [ids, 0, max(1, len(ids) - rng.choice([8, 20, 33]))]
        entries, exp, end = [], [], []
        for rid in list(live):
            ids, p, decode_from = live[rid]
            if len(live) > 1 and rng.random() < 0.2:
                continue                                   # left out of this step, goes on later
            m = 1 if p >= decode_from else min(rng.choice(chunk_sizes), decode_from - p)
            if m == 1 and p < decode_from and decode_from - p >= 2:
                m = 2
            want = list(range(m)) if rng.random() < 0.7 else [m - 1]
            entries.append({"id": rid, "tokens": ids[p:p + m], "want": want})
            exp += [(rid, p + w) for w in want]
            live[rid][1] = p + m
            if p + m == len(ids):
                end.append(rid); del live[rid]
        if not entries:
            continue
        rng.shuffle(entries)
        order = {e["id"]: i for i, e in enumerate(entries)}
        exp_sorted = []
        for e in entries:
            exp_sorted += [x for x in exp if x[0] == e["id"]]
        steps.append({"step": n, "entries": entries, "end": end})
        if exp_sorted:
            expected[n] = exp_sorted
        n += 1
    return steps, expected


def peak_tokens(steps, round_to=64):
    """The most tokens live requests hold at any time, each rounded up to ``round_to``."""
    held, peak = {}, 0
    for s in steps:
        for e in s["entries"]:
            held[e["id"]] = held.get(e["id"], 0) + len(e["tokens"])
        peak = max(peak, sum(-(-v // round_to) * round_to for v in held.values()))
        for rid in s["end"]:
            held.pop(rid, None)
    return peak
