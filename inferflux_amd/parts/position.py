"""Position encodings applied to queries and keys before the cache write.

A position part hands the mixer what its fused kernel needs: ``kernel_args(ctx)`` returns
(style, rotary_dim, cos, sin), the last two being the step's table [T, rotary_dim / 2] of
angle = float(position) * inv_freq[p], computed in float once per step and shared by every
layer with the same constants.  The kernel rotates pair p of every head by it.  A position part
that cannot be expressed this way sets ``needs_apply`` and implements ``apply(q, k, positions)``.

Rotary, split-half ("NeoX") pairing as the reference applies it to qwen2
(runtime/backends/cuda/native/model_loader.h:39-61 chooses the pairing;
cuda_kernels.cu:71-117): pair p joins elements p and p + d/2, f_p = 1 / theta^(2p/d),
(x_p, x_{p+d/2}) <- (x_p cos a - x_{p+d/2} sin a, x_p sin a + x_{p+d/2} cos a).  The reference
evaluates powf per element; here the d/2 frequencies are computed once in double precision
and rounded to float.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from ..kernels import ops
from .base import Part, register_part


class PositionEncoding(Part):
    def kernel_args(self, ctx) -> Tuple[int, int, Optional[torch.Tensor], Optional[torch.Tensor]]:
        return ops.ROPE_NONE, 0, None, None

    def apply(self, q: torch.Tensor, k: Optional[torch.Tensor], positions: torch.Tensor):
        """Transform q [T, nH, d] and k [T, nKV, d] (or None) outside the fused kernel."""
        return q, k

    needs_apply = False


@register_part("position", "none")
class NoPosition(PositionEncoding):
    graph_safe = True

    def __init__(self, head_dim: int = 0):
        self.head_dim = head_dim


@register_part("position", "rotary")
class RotaryPosition(PositionEncoding):
    graph_safe = True

    """``style``: "split_half" pairs (p, p + rot/2); "consecutive" pairs (2p, 2p+1)."""

    STYLES = {"split_half": ops.ROPE_SPLIT_HALF, "consecutive": ops.ROPE_CONSECUTIVE}

    def __init__(self, head_dim: int, theta: float, rotary_dim: Optional[int] = None, style: str = "split_half"):
        self.head_dim = int(head_dim)
        self.rotary_dim = int(rotary_dim) if rotary_dim is not None else self.head_dim
        self.theta = float(theta)
        if style not in self.STYLES:
            raise ValueError(f"rotary style '{style}' unknown (one of {sorted(self.STYLES)})")
        if self.rotary_dim % 2 or not (0 < self.rotary_dim <= self.head_dim):
            raise ValueError(f"rotary_dim {self.rotary_dim} must be even and within head_dim {self.head_dim}")
        self.style = style
        self._inv_freq = {}

    def inv_freq(self, device) -> torch.Tensor:
        key = str(device)
        t = self._inv_freq.get(key)
        if t is None:
            p = torch.arange(self.rotary_dim // 2, dtype=torch.float64)
            t = (1.0 / torch.pow(torch.tensor(self.theta, dtype=torch.float64), 2.0 * p / self.rotary_dim))
            t = t.to(torch.float32).to(device)
            self._inv_freq[key] = t
        return t

    def kernel_args(self, ctx):
        cos, sin = ctx.derived(("rotary_table", self.theta, self.rotary_dim),
                               lambda: ops.rope_table(ctx.positions, self.inv_freq(ctx.device)))
        return self.STYLES[self.style], self.rotary_dim, cos, sin
