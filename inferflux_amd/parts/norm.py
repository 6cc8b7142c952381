"""RMSNorm over the float32 residual stream, fused with the residual add that precedes it.

y = x * rsqrt(mean(x^2) + eps) * w, all in float, one rounding to the activation type at the
end (runtime/backends/cuda/native/cuda_kernels.cu:15-48; with the add: 193-249, 617-671).
"""
from __future__ import annotations

from typing import Dict, Mapping, Optional

import torch

from ..kernels import ops
from .base import Norm, register_part
from .plan import ParamSpec


@register_part("norm", "rmsnorm")
class RMSNorm(Norm):
    graph_safe = True

    def __init__(self, name: str, hidden_size: int, eps: float):
        self.name, self.hidden_size, self.eps = name, int(hidden_size), float(eps)
        self.weight: Optional[torch.Tensor] = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {f"{self.name}.weight": ParamSpec((self.hidden_size,), ("ones",))}

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        self.weight = tensors[f"{self.name}.weight"]

    def rms_params(self):
        return self.weight, self.eps

    def forward(self, residual, delta, out_dtype, rows=None):
        return ops.add_rmsnorm(residual, delta, self.weight, self.eps, out_dtype, rows)
