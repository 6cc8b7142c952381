"""Arrangements of a layer's parts.

"prenorm" is the reference's: norm -> mixer -> add; norm -> feed-forward -> add
(runtime/backends/cuda/native/transformer_forward.cu:1805-1816, 2176-2241, 2260-2271,
2528-2610).  The adds are not done here: each sub-block's output is handed on as a pending
delta, and the norm that follows adds it to the float32 stream in the same kernel that
normalises (the reference's ResidualAddRmsNorm, cuda_kernels.cu:617-671).

For steps of few rows a sub-block that can do so adds its output to the stream in its last product's
epilogue and hands on the next norm's rows up to a factor per row (``ScaledRows``), which the sub-block
after it applies to its first product's sums: the norm between them then needs no kernel.  Parts that
do not declare this are given plain tensors, and a plain delta is taken from them.
"""
from __future__ import annotations

from ..kernels.ops import ScaledRows
from .base import Block, MixerBinding, StreamSink, build_part, register_part
from .plan import LayerSpec


def normed_for(norm, reader, residual, pending, ctx):
    """What ``reader`` is given: the norm of the stream plus ``pending``."""
    if isinstance(pending, ScaledRows):          # the delta is in the stream already
        accepts = getattr(reader, "accepts_scaled_rows", None)
        params = norm.rms_params()
        made_for_this_norm = params is not None and pending.norm_weight is params[0] and pending.eps == params[1]
        if made_for_this_norm and accepts is not None and accepts(pending.shape[0]):
            return pending
        pending = None                           # (rows prepared for another norm are of no use: the stream is)
    return norm.forward(residual, pending, ctx.act_dtype)


def _sink(part, residual, norm):
    if norm is None or not getattr(part, "adds_to_stream", False):
        return None
    params = norm.rms_params()
    return StreamSink(residual, *params) if params is not None else None


@register_part("block", "prenorm")
class PreNormBlock(Block):
    graph_safe = True

    def __init__(self, layer: LayerSpec, hidden_size: int):
        if layer.norm_in is None or layer.norm_post is None or layer.ffn is None or layer.extra:
            raise ValueError(f"layer {layer.prefix}: the prenorm block is two norms, a mixer and a feed-forward, no more and no less")
        self.prefix = layer.prefix
        self.norm_in = build_part("norm", layer.norm_in, hidden_size=hidden_size)
        self.mixer = build_part("mixer", layer.mixer, hidden_size=hidden_size)
        self.norm_post = build_part("norm", layer.norm_post, hidden_size=hidden_size)
        self.ffn = build_part("ffn", layer.ffn, hidden_size=hidden_size)

    def children(self):
        return (self.norm_in, self.mixer, self.norm_post, self.ffn)

    def entry_norm(self):
        return self.norm_in

    def _mixer(self, h, ctx, binding, residual):
        sink = _sink(self.mixer, residual, self.norm_post)
        return self.mixer.forward(h, ctx, binding, sink=sink) if sink is not None else self.mixer.forward(h, ctx, binding)

    def _ffn(self, h, ctx, residual, following):
        sink = _sink(self.ffn, residual, following)
        return self.ffn.forward(h, ctx, sink=sink) if sink is not None else self.ffn.forward(h, ctx)

    def forward(self, residual, pending, ctx, binding: MixerBinding, following=None):
        t = ctx.timer
        if t is None:
            h = normed_for(self.norm_in, self.mixer, residual, pending, ctx)
            delta = self._mixer(h, ctx, binding, residual)
            h = normed_for(self.norm_post, self.ffn, residual, delta, ctx)
            return residual, self._ffn(h, ctx, residual, following)
        t.enter("norm"); h = normed_for(self.norm_in, self.mixer, residual, pending, ctx); t.mark("norm")
        t.enter("mixer"); delta = self._mixer(h, ctx, binding, residual); t.mark("mixer")
        t.enter("norm"); h = normed_for(self.norm_post, self.ffn, residual, delta, ctx); t.mark("norm")
        t.enter("ffn"); out = self._ffn(h, ctx, residual, following); t.mark("ffn")
        return residual, out
