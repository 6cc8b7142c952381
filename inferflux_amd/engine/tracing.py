"""Per-phase timing of a forward pass, for finding where a step's time goes.

Like the reference's PhaseTiming (runtime/backends/cuda/native/transformer_forward.cu:71-131,
enabled there by INFERFLUX_CUDA_PHASE_TIMING=1): the stream is synchronised at every mark and the
wall time since the previous mark is booked to a phase, so the GPU pipeline is serialised while
it is on (the reference measured half the throughput, docs/benchmarks.md:193-199).  For
debugging and profiling only; decode steps are not captured as graphs while it is on.  Each phase
is also a range for the profiler's timeline (roctx through torch.cuda.nvtx, where available), in
the place of the reference's NVTX_SCOPE.
"""
from __future__ import annotations

import sys
import time
from typing import Dict

import torch

PHASES = ("embed", "norm", "mixer", "ffn", "final_norm", "lm_head")


class PhaseTimer:
    def __init__(self, report_every: int = 10, stream=None):
        self.totals: Dict[str, float] = {p: 0.0 for p in PHASES}
        self.step: Dict[str, float] = {}
        self.forwards = 0
        self.report_every = report_every
        self._last = 0.0
        try:
            torch.cuda.nvtx.range_push("inferflux_amd")
            torch.cuda.nvtx.range_pop()
            self._ranges = True
        except Exception:
            self._ranges = False
        self._open = False

    def begin(self) -> None:
        torch.cuda.synchronize()
        self.step = {}
        self._last = time.perf_counter()

    def enter(self, name: str) -> None:
        """Open a profiler range for the phase that starts now."""
        if self._ranges:
            if self._open:
                torch.cuda.nvtx.range_pop()
            torch.cuda.nvtx.range_push(name)
            self._open = True

    def mark(self, name: str) -> None:
        """Book the time since the last mark to ``name``."""
        torch.cuda.synchronize()
        now = time.perf_counter()
        ms = (now - self._last) * 1e3
        self._last = now
        self.step[name] = self.step.get(name, 0.0) + ms
        self.totals[name] = self.totals.get(name, 0.0) + ms

    def end(self, n_layers: int, n_tokens: int) -> None:
        if self._ranges and self._open:
            torch.cuda.nvtx.range_pop()
            self._open = False
        self.forwards += 1
        if self.forwards <= 5 or self.forwards % self.report_every == 0:
            parts = " ".join(f"{k}={v:.2f}" for k, v in self.step.items())
            print(f"[phase_timing] #{self.forwards} L={n_layers} tokens={n_tokens} {parts} "
                  f"total={sum(self.step.values()):.2f} ms", file=sys.stderr, flush=True)


def kernel_trace_summary(csv_path: str, n_steps: int = 16, end_marker: str = "argmax_final") -> str:
    """Per-kernel time per engine step from a ``rocprofv3 --kernel-trace --output-format csv`` file.

    A step ends with the kernel whose name contains ``end_marker`` (the sampler's last kernel); the
    last ``n_steps`` complete steps are averaged.  Returns the text of the table: kernels per step,
    busy time (sum of kernel durations) and span (first start to last end) per step, then one line
    per kernel name.
    """
    import collections
    import csv
    with open(csv_path, newline="") as f:
        rows = sorted(csv.DictReader(f), key=lambda r: int(r["Start_Timestamp"]))
    ends = [i for i, r in enumerate(rows) if end_marker in r["Kernel_Name"]]
    if len(ends) < n_steps + 1:
        raise ValueError(f"{csv_path}: {len(ends)} kernels named *{end_marker}*, need {n_steps + 1}")
    steps = [rows[ends[k - 1] + 1: ends[k] + 1] for k in range(len(ends) - n_steps, len(ends))]
    agg = collections.defaultdict(lambda: [0, 0])
    span = 0
    for st in steps:
        span += int(st[-1]["End_Timestamp"]) - int(st[0]["Start_Timestamp"])
        for r in st:
            a = agg[r["Kernel_Name"][:72]]
            a[0] += int(r["End_Timestamp"]) - int(r["Start_Timestamp"])
            a[1] += 1
    n = len(steps)
    busy = sum(v[0] for v in agg.values())
    lines = [f"steps {n}  kernels/step {sum(v[1] for v in agg.values()) / n:.0f}  busy/step {busy / n / 1e3:.1f} us  "
             f"span/step {span / n / 1e3:.1f} us"]
    for name, (t, c) in sorted(agg.items(), key=lambda kv: -kv[1][0]):
        lines.append(f"{t / n / 1e3:9.1f} us/step  {c / n:6.1f} calls  {t / c / 1e3:8.2f} us each  {name}")
    return "\n".join(lines)


if __name__ == "__main__":
    # python -m inferflux_amd.engine.tracing <kernel_trace.csv> [steps] [end marker]
    print(kernel_trace_summary(sys.argv[1], int(sys.argv[2]) if len(sys.argv) > 2 else 16,
                               sys.argv[3] if len(sys.argv) > 3 else "argmax_final"))
