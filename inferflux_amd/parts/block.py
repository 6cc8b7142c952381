"""Arrangements of a layer's parts.

"prenorm" is the reference's: norm -> mixer -> add; norm -> feed-forward -> add
(runtime/backends/cuda/native/transformer_forward.cu:1805-1816, 2176-2241, 2260-2271,
2528-2610).  The adds are not done here: each sub-block's output is handed on as a pending
delta, and the norm that follows adds it to the float32 stream in the same kernel that
normalises (the reference's ResidualAddRmsNorm, cuda_kernels.cu:617-671).
"""
from __future__ import annotations

from .base import Block, MixerBinding, build_part, register_part
from .plan import LayerSpec


@register_part("block", "prenorm")
class PreNormBlock(Block):
    graph_safe = True

    def __init__(self, layer: LayerSpec, hidden_size: int):
        self.prefix = layer.prefix
        self.norm_in = build_part("norm", layer.norm_in, hidden_size=hidden_size)
        self.mixer = build_part("mixer", layer.mixer, hidden_size=hidden_size)
        self.norm_post = build_part("norm", layer.norm_post, hidden_size=hidden_size)
        self.ffn = build_part("ffn", layer.ffn, hidden_size=hidden_size)

    def children(self):
        return (self.norm_in, self.mixer, self.norm_post, self.ffn)

    def forward(self, residual, pending, ctx, binding: MixerBinding):
        t = ctx.timer
        if t is None:
            h = self.norm_in.forward(residual, pending, ctx.act_dtype)
            delta = self.mixer.forward(h, ctx, binding)
            h = self.norm_post.forward(residual, delta, ctx.act_dtype)
            return residual, self.ffn.forward(h, ctx)
        t.enter("norm"); h = self.norm_in.forward(residual, pending, ctx.act_dtype); t.mark("norm")
        t.enter("mixer"); delta = self.mixer.forward(h, ctx, binding); t.mark("mixer")
        t.enter("norm"); h = self.norm_post.forward(residual, delta, ctx.act_dtype); t.mark("norm")
        t.enter("ffn"); out = self.ffn.forward(h, ctx); t.mark("ffn")
        return residual, out
