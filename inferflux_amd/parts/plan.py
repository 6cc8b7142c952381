"""The data that describes a model: which parts make each layer, and in which order layers run.

A ``ModelPlan`` is produced from a typed config by the architecture's plan builder and
is all the generic model needs: it names parts by their registry name with their sizes
and constants as arguments, layer by layer, so layers of one model may differ in mixer,
feed-forward, norm or window.  The run order (``schedule``) is a list too: it may name a
layer twice, and an entry may read the cache that another entry writes.
"""
from __future__ import annotations

import dataclasses
from typing import Any, Dict, Optional, Tuple


@dataclasses.dataclass(frozen=True)
class PartSpec:
    """A part by registry name, with its constructor arguments (sizes and constants)."""
    kind: str
    args: Dict[str, Any] = dataclasses.field(default_factory=dict)


@dataclasses.dataclass(frozen=True)
class LayerSpec:
    """One layer: an arrangement (``block``) of parts.  The arrangement decides which of them it uses: the
    built-in "prenorm" block takes two norms, a mixer and a feed-forward; another block may leave the norms or
    the feed-forward out (None) and take further parts by name from ``extra`` (category, spec): a third and
    fourth norm, a second feed-forward, ...  Every layer has a mixer: it is what owns cache and state.

    ``prefix`` is the tensor-name prefix of the layer's weights ("model.layers.3").
    """
    prefix: str
    block: PartSpec
    norm_in: Optional[PartSpec]
    mixer: PartSpec
    norm_post: Optional[PartSpec] = None
    ffn: Optional[PartSpec] = None
    extra: Tuple[Tuple[str, str, PartSpec], ...] = ()      # (name, category, spec) of further parts

    def extra_part(self, name: str) -> Tuple[str, PartSpec]:
        for n, category, spec in self.extra:
            if n == name:
                return category, spec
        raise KeyError(f"layer {self.prefix}: no extra part named '{name}' (has: {[n for n, _, _ in self.extra]})")


@dataclasses.dataclass(frozen=True)
class ScheduleEntry:
    """One execution of a layer.

    ``layer`` indexes ``ModelPlan.layers``.  ``cache_from`` is None when the entry's mixer
    owns a cache of its own, or the index of an earlier schedule entry whose cache this
    entry's mixer reads without writing.
    """
    layer: int
    cache_from: Optional[int] = None


@dataclasses.dataclass(frozen=True)
class ModelPlan:
    vocab_size: int
    hidden_size: int
    max_position: int
    embedding: PartSpec
    layers: Tuple[LayerSpec, ...]
    schedule: Tuple[ScheduleEntry, ...]
    final_norm: PartSpec
    lm_head: PartSpec
    eos_token_ids: Tuple[int, ...] = ()      # every token id that ends a request (a model may name several)

    def validate(self) -> None:
        if not self.layers:
            raise ValueError("plan has no layers")
        for i, e in enumerate(self.schedule):
            if not (0 <= e.layer < len(self.layers)):
                raise ValueError(f"schedule[{i}] names layer {e.layer}, plan has {len(self.layers)}")
            if e.cache_from is not None:
                if not (0 <= e.cache_from < i):
                    raise ValueError(f"schedule[{i}].cache_from={e.cache_from} must name an earlier entry")
                if self.schedule[e.cache_from].cache_from is not None:
                    raise ValueError(f"schedule[{i}].cache_from={e.cache_from} names an entry that owns no cache")


@dataclasses.dataclass(frozen=True)
class ParamSpec:
    """A tensor a part expects in the model file.

    ``init`` is how the random-weights mode fills it: ("normal", std), ("ones",) or
    ("zeros",).  ``integer`` tensors are kept as int32; floating tensors follow the
    engine's dtype rule (see weights.loader).
    """
    shape: Tuple[int, ...]
    init: Tuple = ("normal", 0.02)
    optional: bool = False
    integer: bool = False


@dataclasses.dataclass(frozen=True)
class CacheSpec:
    """What a mixer keeps per token: keys of ``n_kv_heads`` x ``head_dim`` and values of ``n_kv_heads`` x
    ``v_head_dim`` (None: as wide as the keys).

    ``window`` is None when every past token stays readable, or the number of most recent
    positions (the current one included) that the mixer reads; older pages are given back.
    """
    n_kv_heads: int
    head_dim: int
    window: Optional[int] = None
    v_head_dim: Optional[int] = None

    @property
    def k_dim(self) -> int:
        return self.head_dim

    @property
    def v_dim(self) -> int:
        return self.head_dim if self.v_head_dim is None else self.v_head_dim

    def bytes_per_token(self, element_size: int) -> int:
        return self.n_kv_heads * (self.k_dim + self.v_dim) * element_size


@dataclasses.dataclass(frozen=True)
class StateSpec:
    """Fixed-size per-request state of a mixer: one tensor of ``shape`` per live request,
    zero when the request starts."""
    shape: Tuple[int, ...]
    dtype: str = "float32"
