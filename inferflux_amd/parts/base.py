"""Interfaces of the parts a layer is made of, and the registry that finds them by name.

A part is built from its sizes and constants alone; it never sees the model's config and does
not know which model it is in.  It declares the tensors it expects under its weight prefix
(``param_specs``), receives them once (``load``), and then runs on a step's rows.

Categories and what each must provide beyond ``param_specs`` / ``load``:

  norm      forward(residual, delta, rows=None) -> normalised rows in the activation type.
            ``residual`` is the float32 stream [T, H]; ``delta`` (or None) is first added to it
            in place.  With ``rows`` only those rows are returned and nothing is written.
  position  prepares what the mixer's kernels need to encode positions (see parts/position.py);
            a position part may also transform q and k itself through ``apply(q, k, positions)``.
  mixer     forward(h, ctx, binding) -> delta [T, H].  ``cache_spec()`` says what it keeps per
            token (or None), ``state_spec()`` what fixed-size state it keeps per request (or
            None).  ``binding`` carries the cache tensors / state tensor the model allocated for
            this execution of the layer.
  ffn       forward(h, ctx) -> delta [T, H].
  block     the arrangement: forward(residual, pending, ctx, binding) -> (residual, pending),
            where ``pending`` is a delta not yet added to the stream (the next norm adds it).
  embedding forward(ctx) -> float32 stream [T, H] of the step's rows (``ctx.token_ids``, and whatever else of the
            step it needs: ``ctx.positions`` for a learned position table, ...).
  head      forward(normalised rows) -> float32 logits [R, V].

A norm's kernel can be saved for steps of few rows, where a launch costs as much as the work.  This is
optional for every part; one that declares nothing is run as above.

  norm      ``rms_params()`` -> (weight, eps) if the norm is x * rsqrt(mean(x^2) + eps) * weight, else None.
            Such a norm's forward also takes ``SliceSums`` (a product left as partial sums; kernels/ops.py) for
            its delta, as ``ops.add_rmsnorm`` does.
  mixer,    ``adds_to_stream`` True: forward takes ``sink=StreamSink(stream, weight, eps)`` (or None) and may
  ffn       then add its result to the stream itself and return ``ScaledRows`` (the rows the norm that follows
            would give, up to a factor per row; kernels/ops.py) instead of a delta, or return its delta as
            ``SliceSums``.
            ``accepts_scaled_rows(n_rows)`` True: forward takes ``ScaledRows`` for h.
  block     ``entry_norm()`` -> the norm that first reads the stream, if ``pending`` may be ``ScaledRows`` made
            for it; forward then takes ``following=`` the next block's entry norm (or None; for the last block the
            final norm, in steps that want every row's logits).
  embedding ``prepares_norm_rows`` True: forward takes ``norm=`` the first block's entry norm and may return
            (stream, ``ScaledRows`` made for that norm).
  head      ``accepts_scaled_rows(n_rows)`` True: forward takes ``ScaledRows`` for the normalised rows.
"""
from __future__ import annotations

import dataclasses
from typing import Callable, Dict, Mapping, Optional

import torch

from .plan import CacheSpec, ParamSpec, PartSpec, StateSpec

_REGISTRY: Dict[str, Dict[str, Callable]] = {}
CATEGORIES = ("norm", "position", "mixer", "ffn", "block", "embedding", "head")


def register_part(category: str, name: str):
    """Class decorator: make ``cls`` buildable from ``PartSpec(kind=name)`` in ``category``."""
    if category not in CATEGORIES:
        raise ValueError(f"unknown part category '{category}' (one of {CATEGORIES})")

    def deco(cls):
        table = _REGISTRY.setdefault(category, {})
        if name in table and table[name] is not cls:
            raise ValueError(f"{category} part '{name}' is already registered")
        table[name] = cls
        return cls

    return deco


def build_part(category: str, spec: PartSpec, **context) -> "Part":
    """Build the part ``spec`` names.  ``context`` holds what the surrounding structure knows
    (``prefix`` of the weight names, ``hidden_size``); the part's own sizes are in ``spec.args``."""
    table = _REGISTRY.get(category, {})
    if spec.kind not in table:
        raise KeyError(f"no {category} part named '{spec.kind}'; registered: {sorted(table)}")
    return table[spec.kind](**context, **spec.args)


def registered_parts(category: str):
    return sorted(_REGISTRY.get(category, {}))


class Part:
    """Base of all parts.

    ``graph_safe`` says that ``forward`` reads a step's metadata only from the context's device
    tensors and launches the same kernels with the same grid for every step of one layout
    (``StepContext.layout_key``), so that a decode step may be captured once and replayed.  A part
    that loops on the host over ``ctx.h_*`` arrays must leave it False; a model with such a part
    runs every step eagerly.
    """

    graph_safe = False

    def param_specs(self) -> Dict[str, ParamSpec]:
        """Full tensor names this part reads from the model file."""
        return {}

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        """Take the part's tensors (already on the device, stored by the loader's rule)."""

    def children(self):
        return ()


@dataclasses.dataclass
class LayerCache:
    """The cache tensors of one schedule entry: K [pages, kv heads, page_size, d] and
    V [pages, kv heads, dv, page_size] (dv = d unless the mixer's ``CacheSpec`` says otherwise), and the cache
    group whose block tables index them."""
    k: torch.Tensor
    v: torch.Tensor
    group: int
    page_size: int


@dataclasses.dataclass
class MixerBinding:
    """What one execution of a layer's mixer works on.

    ``cache`` is None for a mixer without cache.  ``writes_cache`` is False when the entry
    reads the cache another entry owns.  ``state`` is the [slots, *shape] tensor of the
    mixer's per-request state, or None.
    """
    cache: Optional[LayerCache] = None
    writes_cache: bool = True
    state: Optional[torch.Tensor] = None


@dataclasses.dataclass
class StreamSink:
    """Where a mixer or feed-forward may add its result itself: the float32 stream, and the weight and eps
    of the RMS norm that reads the stream next."""
    stream: torch.Tensor
    norm_weight: torch.Tensor
    eps: float


class Mixer(Part):
    adds_to_stream = False

    def accepts_scaled_rows(self, n_rows: int) -> bool:
        return False

    def cache_spec(self) -> Optional[CacheSpec]:
        return None

    def state_spec(self) -> Optional[StateSpec]:
        return None

    def forward(self, h: torch.Tensor, ctx, binding: MixerBinding) -> torch.Tensor:
        raise NotImplementedError


class FeedForward(Part):
    adds_to_stream = False

    def accepts_scaled_rows(self, n_rows: int) -> bool:
        return False

    def forward(self, h: torch.Tensor, ctx) -> torch.Tensor:
        raise NotImplementedError


class Norm(Part):
    def rms_params(self):
        return None

    def forward(self, residual: torch.Tensor, delta: Optional[torch.Tensor], out_dtype: torch.dtype,
                rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        raise NotImplementedError


class Block(Part):
    def entry_norm(self) -> Optional[Norm]:
        return None

    def forward(self, residual, pending, ctx, binding: MixerBinding):
        raise NotImplementedError
