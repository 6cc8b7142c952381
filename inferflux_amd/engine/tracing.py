"""Per-phase timing of a forward pass, for finding where a step's time goes.

Like the reference's PhaseTiming (runtime/backends/cuda/native/transformer_forward.cu:71-131,
enabled there by INFERFLUX_CUDA_PHASE_TIMING=1), which synchronises the stream at every mark and
measured half the throughput with it on (docs/benchmarks.md:193-199).  Here a mark records an event on
the stream and the step is waited for once, at its end; the time between two events is booked to the
phase that the later one names.  The GPU's work is not serialised against the host, so the figures are
GPU time, including whatever the GPU waited for the host inside the phase (eager steps of few rows).
Decode steps are not captured as graphs while it is on.  Each phase is also a range for the profiler's
timeline (roctx through torch.cuda.nvtx, where available), in the place of the reference's NVTX_SCOPE.

Blocks mark "norm", "mixer" and "ffn"; the attention mixer and the gated feed-forward mark their own
stages before that ("mixer.qkv", "mixer.attention", "ffn.gate_up"; what is left for the block's mark
is the output projection and the down projection).
"""
from __future__ import annotations

import sys
from typing import Dict, List, Tuple

import torch

PHASES = ("embed", "norm", "mixer.qkv", "mixer.attention", "mixer", "ffn.gate_up", "ffn", "final_norm", "lm_head")


class PhaseTimer:
    def __init__(self, report_every: int = 10, quiet: bool = False):
        self.totals: Dict[str, float] = {p: 0.0 for p in PHASES}     # ms, over all forwards
        self.step: Dict[str, float] = {}                             # ms, the last forward
        self.forwards = 0
        self.report_every = report_every
        self.quiet = quiet
        self._marks: List[Tuple[str, torch.cuda.Event]] = []
        self._start = None
        try:
            torch.cuda.nvtx.range_push("inferflux_amd")
            torch.cuda.nvtx.range_pop()
            self._ranges = True
        except Exception:
            self._ranges = False
        self._open = False

    def _event(self) -> torch.cuda.Event:
        e = torch.cuda.Event(enable_timing=True)
        e.record()
        return e

    def begin(self) -> None:
        self._marks = []
        self._start = self._event()

    def enter(self, name: str) -> None:
        """Open a profiler range for the phase that starts now."""
        if self._ranges:
            if self._open:
                torch.cuda.nvtx.range_pop()
            torch.cuda.nvtx.range_push(name)
            self._open = True

    def mark(self, name: str) -> None:
        """Book the GPU time since the last mark to ``name``."""
        self._marks.append((name, self._event()))

    def end(self, n_layers: int, n_tokens: int) -> None:
        if self._ranges and self._open:
            torch.cuda.nvtx.range_pop()
            self._open = False
        self.step = {}
        if self._marks:
            self._marks[-1][1].synchronize()
            last = self._start
            for name, ev in self._marks:
                ms = last.elapsed_time(ev)
                last = ev
                self.step[name] = self.step.get(name, 0.0) + ms
                self.totals[name] = self.totals.get(name, 0.0) + ms
        self.forwards += 1
        if not self.quiet and (self.forwards <= 5 or self.forwards % self.report_every == 0):
            parts = " ".join(f"{k}={v:.2f}" for k, v in self.step.items())
            print(f"[phase_timing] #{self.forwards} L={n_layers} tokens={n_tokens} {parts} "
                  f"total={sum(self.step.values()):.2f} ms", file=sys.stderr, flush=True)

    def shares(self) -> Dict[str, float]:
        """Each phase's share of the time booked so far."""
        total = sum(self.totals.values())
        return {k: v / total for k, v in self.totals.items() if v > 0.0} if total > 0 else {}


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
