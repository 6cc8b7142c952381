"""Replays traces through bin/trace_run as a user would (a subprocess, files on disk) and compares
every logits row with the plain implementation's whole-sequence logits: whole requests, a prefill
with the last 32 tokens one by one, portions of changing size, and mixed steps with so few pages
that they are used again.  In 32-bit and in bfloat16, for each tiny configuration."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import traces
from conftest import REL_TOL, tol, ROOT, TINY, plain_logits, rel_err, seeded_ids

pytestmark = pytest.mark.gpu

LENGTHS = {"A": [45, 70, 96, 130, 33, 64, 120], "B": [1, 17, 64, 100, 250, 40], "C": [45, 90, 33, 140, 64, 100]}


def replay(folder, dtype, steps, out_dir, max_tokens):
    proc = subprocess.Popen([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype,
                             "--out", out_dir, "--max-tokens", str(max_tokens)],
                            stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)
    try:
        for s in steps:
            proc.stdin.write(json.dumps(s) + "\n")
            proc.stdin.flush()
            line = proc.stdout.readline().strip()          # the next step may come only after "done"
            assert line == f"done {s['step']}", f"trace_run said {line!r} for step {s['step']}"
        proc.stdin.close()
        assert proc.wait(timeout=120) == 0
    finally:
        if proc.poll() is None:
            proc.kill()


def check(folder, dtype, seqs, expected, out_dir, vocab, name):
    worst = 0.0
    for step, rows in expected.items():
        got = np.fromfile(os.path.join(out_dir, f"{step}.f32"), dtype="<f4")
        assert got.size == len(rows) * vocab, f"step {step}: {got.size} floats for {len(rows)} rows"
        got = torch.from_numpy(got.reshape(len(rows), vocab))
        want = torch.stack([plain_logits(folder, seqs[rid])[p] for rid, p in rows])
        assert torch.isfinite(got).all(), f"step {step}"
        e = rel_err(got, want)
        assert e < tol(dtype, name), f"step {step} rows {rows[:4]}...: relative error {e:.3g}"
        worst = max(worst, e)
    return worst


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(TINY))
def test_all_cuttings_match_the_plain_model(name, dtype, sharp_folders, tmp_path):
    folder, vocab = sharp_folders[name, dtype], TINY[name]["vocab_size"]
    seqs = {f"r{i}": seeded_ids(300 + i, n, vocab) for i, n in enumerate(LENGTHS[name])}
    # One process replays all four ways, one after the other, from one small pool: requests of a later
    # way get the pages that earlier ones gave back.
    all_steps, all_expected, offset = [], {}, 0
    for build in (traces.whole, traces.prefill_then_decode, traces.portions, lambda s: traces.mixed(s, seed=len(name))):
        steps, expected = build(seqs)
        for s in steps:
            s["step"] += offset
        all_expected.update({k + offset: v for k, v in expected.items()})
        all_steps += steps
        offset += len(steps)
    max_tokens = traces.peak_tokens(all_steps)
    assert max_tokens <= 4 * 256
    out = str(tmp_path / "out")
    replay(folder, dtype, all_steps, out, max_tokens)
    files = sorted(int(f[:-4]) for f in os.listdir(out))
    assert files == sorted(all_expected), "a logits file for every step that wants something, and no other"
    check(folder, dtype, seqs, all_expected, out, vocab, name)
