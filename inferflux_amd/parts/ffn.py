"""SwiGLU feed-forward: down( silu(gate(x)) * up(x) ), no biases.

g = h Wg^T, u = h Wu^T, a = g / (1 + exp(-g)) * u in float, delta = a Wd^T
(runtime/backends/cuda/native/transformer_forward.cu:2383-2419, 2487-2494, 2528-2547;
cuda_kernels.cu:139-151).  The reference runs gate and up as two products; here the two
matrices are merged at load time into one [2I, H] matrix whose rows alternate gate_i, up_i, so
that one product yields both and the kernel that holds a gate value also holds its up value
(the activation is then the product's epilogue).  This changes nothing in the arithmetic of
any output element.
"""
from __future__ import annotations

from typing import Dict, Mapping

import torch

from ..kernels import ops
from .base import FeedForward, register_part
from .plan import ParamSpec


def concat_weights(parts):
    """Stack matrices along the output axis; mixed storage types are widened to float32."""
    if len({p.dtype for p in parts}) > 1:
        parts = [p.float() for p in parts]
    return torch.cat(list(parts), dim=0).contiguous()


@register_part("ffn", "swiglu")
class SwiGLU(FeedForward):
    graph_safe = True

    def __init__(self, name: str, hidden_size: int, intermediate_size: int, init_std: float = 0.02):
        self.name, self.hidden_size, self.intermediate_size = name, int(hidden_size), int(intermediate_size)
        self.init_std = init_std
        self.w_gate_up = None
        self.w_down = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        H, I, s = self.hidden_size, self.intermediate_size, ("normal", self.init_std)
        return {
            f"{self.name}.gate_proj.weight": ParamSpec((I, H), s),
            f"{self.name}.up_proj.weight": ParamSpec((I, H), s),
            f"{self.name}.down_proj.weight": ParamSpec((H, I), s),
        }

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        g, u = tensors[f"{self.name}.gate_proj.weight"], tensors[f"{self.name}.up_proj.weight"]
        if g.dtype != u.dtype:
            g, u = g.float(), u.float()
        self.w_gate_up = ops.prepare_linear(
            torch.stack([g, u], dim=1).reshape(2 * self.intermediate_size, self.hidden_size).contiguous())
        self.w_down = ops.prepare_linear(tensors[f"{self.name}.down_proj.weight"])

    adds_to_stream = True

    def accepts_scaled_rows(self, n_rows: int) -> bool:
        return ops.takes_scaled_rows(n_rows, self.w_gate_up)

    def forward(self, h, ctx, sink=None):
        a = ops.linear_swiglu(h, self.w_gate_up)
        if ctx.timer is not None:
            ctx.timer.mark("ffn.gate_up")
        if sink is not None and ops.adds_into_stream(a.shape[0], self.w_down, sink.norm_weight):
            return ops.linear_into_stream(a, self.w_down, sink.stream, sink.norm_weight, sink.eps)
        return ops.linear(a, self.w_down, keep_slices=sink is not None)   # an RMS norm's kernel adds partial sums itself
