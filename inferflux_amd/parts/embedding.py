"""Token embedding and the output head.

Embedding: x[t] = E[id[t]], no scaling, widened to the float32 stream
(runtime/backends/cuda/native/cuda_kernels.cu:674-689).  Head: logits = h Wlm^T in float; the
reference rounds logits to the activation type before widening them
(transformer_forward.cu:2686-2699), which is not copied: logits are produced in float32.
A tied head uses the embedding table (the reference ties when lm_head.weight is absent,
weight_map.cpp:33-37; here the configuration says so and the file is checked against it).
"""
from __future__ import annotations

from typing import Dict, Mapping, Optional

import torch

from ..kernels import ops
from .base import Part, register_part
from .plan import ParamSpec


@register_part("embedding", "token_embedding")
class TokenEmbedding(Part):
    graph_safe = True

    def __init__(self, name: str, vocab_size: int, hidden_size: int, init_std: float = 0.02):
        self.name, self.vocab_size, self.hidden_size, self.init_std = name, int(vocab_size), int(hidden_size), init_std
        self.table: Optional[torch.Tensor] = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {f"{self.name}.weight": ParamSpec((self.vocab_size, self.hidden_size), ("normal", self.init_std))}

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        self.table = tensors[f"{self.name}.weight"]

    prepares_norm_rows = True

    def forward(self, ctx, norm=None):
        """The float32 stream of the step's tokens.  Told the norm that reads the stream first (``norm``), a step of few
        tokens in bfloat16 also gets that norm's rows up to a factor per row, (stream, ``ops.ScaledRows``), which
        saves the norm a kernel of its own where the layer's first product takes such rows."""
        params = norm.rms_params() if norm is not None else None
        if (params is not None and 0 < ctx.n_tokens <= 16 and ctx.act_dtype == torch.bfloat16
                and params[0].dtype == torch.bfloat16):
            return ops.embedding_scaled(ctx.token_ids, self.table, params[0], params[1])
        return ops.embedding(ctx.token_ids, self.table)


@register_part("head", "linear_head")
class LinearHead(Part):
    graph_safe = True

    """``tied_to`` names the tensor (the embedding table) a tied head shares; None for its own."""

    def __init__(self, name: str, vocab_size: int, hidden_size: int, tied_to: Optional[str] = None, init_std: float = 0.02):
        self.name, self.vocab_size, self.hidden_size, self.tied_to, self.init_std = name, int(vocab_size), int(hidden_size), tied_to, init_std
        self.weight: Optional[ops.LinearWeight] = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        if self.tied_to:
            return {}
        return {f"{self.name}.weight": ParamSpec((self.vocab_size, self.hidden_size), ("normal", self.init_std))}

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        self.weight = ops.prepare_linear(tensors[self.tied_to or f"{self.name}.weight"])

    def accepts_scaled_rows(self, n_rows: int) -> bool:
        return ops.takes_scaled_rows(n_rows, self.weight)

    def forward(self, h) -> torch.Tensor:
        return ops.linear(h, self.weight, out_dtype=torch.float32)
