"""Chooses the attention kernel for a step.

Every choice computes the same function (causal, optionally windowed, grouped-query attention
over the paged cache); they differ in speed and in which sizes they accept.
"""
from __future__ import annotations

from typing import Optional

import torch

from . import ops


def paged_attention(q: torch.Tensor, cache, ctx, window: Optional[int], scale: float) -> torch.Tensor:
    """q [T, nH, d] of this step's rows against ``cache`` (a LayerCache); returns [T, nH*d]."""
    return ops.attention_plain(q, cache.k, cache.v, ctx.row_req, ctx.positions, ctx.block_table(cache.group),
                               window, scale)
