"""Grouped-query attention over the paged cache, with q/k/v bias, a position part and an
optional window.

Reference order (runtime/backends/cuda/native/transformer_forward.cu:1944-2135, 2145-2241):
q, k, v = h Wq^T + bq, h Wk^T + bk, h Wv^T + bv; position encoding of q and k; k and v are
written to the cache at the token's position; causal attention of head h over kv head
h / (nH / nKV) with scale 1/sqrt(d) applied after the dot product; delta = attn Wo^T.
The three projections are concatenated at load time into one [(nH + 2 nKV) d, H] product;
the bias is added in float inside the rotary kernel (the reference rounds the product to the
activation type first and adds the bias afterwards, cuda_kernels.cu:518-527).

An execution that reads another entry's cache (binding.writes_cache False) projects and
encodes only its queries.
"""
from __future__ import annotations

import math
from typing import Dict, Mapping, Optional

import torch

from ..kernels import ops
from ..kernels.attention import paged_attention
from .base import Mixer, MixerBinding, build_part, register_part
from .ffn import concat_weights
from .plan import CacheSpec, ParamSpec, PartSpec


@register_part("mixer", "paged_attention")
class PagedAttention(Mixer):
    graph_safe = True

    def __init__(self, name: str, hidden_size: int, n_heads: int, n_kv_heads: int, head_dim: int,
                 position: PartSpec, bias: bool = True, window: Optional[int] = None,
                 scale: Optional[float] = None, init_std: float = 0.02, v_head_dim: Optional[int] = None):
        """``v_head_dim``: the width of a value head where it differs from ``head_dim`` (such a layer runs on the
        kernels that take both widths: the plain attention kernel and the unfused projection path)."""
        if n_heads % n_kv_heads:
            raise ValueError(f"{name}: {n_heads} query heads are not a multiple of {n_kv_heads} kv heads")
        self.name, self.hidden_size = name, int(hidden_size)
        self.n_heads, self.n_kv_heads, self.head_dim = int(n_heads), int(n_kv_heads), int(head_dim)
        self.v_head_dim = int(v_head_dim) if v_head_dim else self.head_dim
        self.bias, self.window, self.init_std = bool(bias), (int(window) if window else None), init_std
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(self.head_dim)
        self.position = build_part("position", position)
        self.w_qkv = self.b_qkv = self.w_o = self._w_q = None

    def cache_spec(self) -> CacheSpec:
        return CacheSpec(self.n_kv_heads, self.head_dim, self.window,
                         self.v_head_dim if self.v_head_dim != self.head_dim else None)

    def param_specs(self) -> Dict[str, ParamSpec]:
        H, d, dv, s = self.hidden_size, self.head_dim, self.v_head_dim, ("normal", self.init_std)
        out = {
            f"{self.name}.q_proj.weight": ParamSpec((self.n_heads * d, H), s),
            f"{self.name}.k_proj.weight": ParamSpec((self.n_kv_heads * d, H), s),
            f"{self.name}.v_proj.weight": ParamSpec((self.n_kv_heads * dv, H), s),
            f"{self.name}.o_proj.weight": ParamSpec((H, self.n_heads * dv), s),
        }
        if self.bias:
            out[f"{self.name}.q_proj.bias"] = ParamSpec((self.n_heads * d,), s)
            out[f"{self.name}.k_proj.bias"] = ParamSpec((self.n_kv_heads * d,), s)
            out[f"{self.name}.v_proj.bias"] = ParamSpec((self.n_kv_heads * dv,), s)
        return out

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        n = self.name
        self.w_qkv = self._prepare_qkv(concat_weights([tensors[f"{n}.{p}_proj.weight"] for p in "qkv"]),
                                       self.n_heads + 2 * self.n_kv_heads)
        self.b_qkv = concat_weights([tensors[f"{n}.{p}_proj.bias"] for p in "qkv"]) if self.bias else None
        self.w_o = ops.prepare_linear(tensors[f"{n}.o_proj.weight"])
        self._w_q = None

    def _prepare_qkv(self, weight: torch.Tensor, heads: int):
        """The projection's weight with its decode copy; for head sizes that are multiples of 32 the copy's
        row tiles are ordered so that the fused projection + rotation kernel finds both halves of a rotation
        pair in one lane (plain products read the same copy through the order)."""
        order = None
        if self.head_dim % 32 == 0 and self.v_head_dim == self.head_dim and weight.is_cuda and weight.dtype == torch.bfloat16:
            order = torch.tensor(ops.pair_tile_order(heads, self.head_dim), dtype=torch.int32, device=weight.device)
        return ops.prepare_linear(weight, order)

    adds_to_stream = True

    def accepts_scaled_rows(self, n_rows: int) -> bool:
        return not self.position.needs_apply and ops.takes_scaled_rows(n_rows, self.w_qkv)

    def _project_out(self, out, sink):
        if sink is not None and ops.adds_into_stream(out.shape[0], self.w_o, sink.norm_weight):
            return ops.linear_into_stream(out, self.w_o, sink.stream, sink.norm_weight, sink.eps)
        return ops.linear(out, self.w_o, keep_slices=sink is not None)   # an RMS norm's kernel adds partial sums itself

    def forward(self, h, ctx, binding: MixerBinding, sink=None):
        cache = binding.cache
        nH, d = self.n_heads, self.head_dim
        nKV = self.n_kv_heads if binding.writes_cache else 0
        width = (nH + nKV) * d + nKV * self.v_head_dim
        style, rotary_dim, cos, sin = self.position.kernel_args(ctx)
        w, b = self.w_qkv, self.b_qkv
        if not binding.writes_cache:  # only the queries: the first nH*d rows of the fused matrix
            if self._w_q is None:
                self._w_q = self._prepare_qkv(w.rows[:width], self.n_heads)
            w, b = self._w_q, (b[:width] if b is not None else None)
        slots = ctx.write_slots(cache.group) if binding.writes_cache else None
        t = ctx.timer
        if (style == ops.ROPE_SPLIT_HALF and rotary_dim == d and w.order is not None and h.dtype == torch.bfloat16
                and h.shape[0] <= 16 and not self.position.needs_apply):
            # few tokens: the rotation and the cache write are the projection's epilogue
            q = ops.qkv_rope_append(h, w, b, slots, cos, sin, nH, nKV, d, cache.k if slots is not None else None,
                                    cache.v if slots is not None else None, cache.page_size)
            if t is not None:
                t.mark("mixer.qkv")
            a = paged_attention(q, cache, ctx, self.window, self.scale)
            if t is not None:
                t.mark("mixer.attention")
            return self._project_out(a, sink)
        qkv = ops.linear(h, w, keep_slices=not self.position.needs_apply)     # the rotary kernel adds partial sums itself
        if self.position.needs_apply:
            qkv, b = self._encode_outside(qkv, b, ctx, nKV), None
        q = ops.rope_append(qkv, b, slots, cos, sin, style, rotary_dim, nH, nKV, d,
                            cache.k if slots is not None else None, cache.v if slots is not None else None,
                            cache.page_size, self.v_head_dim)
        if t is not None:
            t.mark("mixer.qkv")
        a = paged_attention(q, cache, ctx, self.window, self.scale)
        if t is not None:
            t.mark("mixer.attention")
        return self._project_out(a, sink)

    def _encode_outside(self, qkv, bias, ctx, nKV):
        """For a position part that transforms q and k itself: add the bias, let the part encode,
        and hand the kernel rows it only has to copy."""
        nH, d, T = self.n_heads, self.head_dim, qkv.shape[0]
        if bias is not None:
            qkv = (qkv.float() + bias.float()).to(qkv.dtype)
        q = qkv[:, : nH * d].reshape(T, nH, d)
        k = qkv[:, nH * d: (nH + nKV) * d].reshape(T, nKV, d) if nKV else None
        q, k = self.position.apply(q, k, ctx.positions)
        cols = [q.reshape(T, nH * d)]
        if nKV:
            cols += [k.reshape(T, nKV * d), qkv[:, (nH + nKV) * d:]]
        return torch.cat(cols, dim=1).contiguous()
