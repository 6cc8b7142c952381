"""Device memory of the cache: the K/V page tensors of every cache-owning schedule entry and the
per-request state tensors, laid out from what the model's mixers declare.

K pages are [page][kv head][offset][d] (a key's elements contiguous, as the score needs them);
V pages are [page][kv head][dv][offset] (a page's values of one element contiguous, as the
weighted sum needs them).  Validity is defined by block tables and lengths, so pages are never
cleared when they change hands; they are zero when first allocated so that a masked key can
never contribute a NaN.  The reference keeps one contiguous [max_seq][nKV*d] slab per sequence
slot, zero-filled, and clears a slot when it is reused
(runtime/backends/cuda/native/kv_cache_gpu.cu:33-35, 49, 107-120).
"""
from __future__ import annotations

from typing import Dict, List, Optional, Tuple

import torch

from ..parts.base import LayerCache, MixerBinding
from .manager import CacheManager, GroupSpec

_STATE_DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16, "int32": torch.int32}


def plan_groups(schedule, mixers) -> Tuple[List[GroupSpec], Dict[int, int]]:
    """Group the cache-owning schedule entries by what they keep (everything, or a window).

    ``mixers[i]`` is the mixer schedule entry i runs.  Returns the groups and, for every entry
    that touches a cache (its own or another's), the group it belongs to.
    """
    by_window: Dict[Optional[int], List[int]] = {}
    for i, e in enumerate(schedule):
        spec = mixers[i].cache_spec()
        if spec is None or e.cache_from is not None:
            continue
        by_window.setdefault(spec.window, []).append(i)
    keys = sorted(by_window, key=lambda w: (w is not None, w or 0))
    groups = [GroupSpec(window=w, entries=tuple(by_window[w])) for w in keys]
    entry_group = {i: g for g, spec in enumerate(groups) for i in spec.entries}
    for i, e in enumerate(schedule):
        if e.cache_from is not None and mixers[i].cache_spec() is not None:
            owner = mixers[e.cache_from].cache_spec()
            mine = mixers[i].cache_spec()
            if owner is None or (owner.n_kv_heads, owner.k_dim, owner.v_dim) != (mine.n_kv_heads, mine.k_dim, mine.v_dim):
                raise ValueError(f"schedule[{i}] reads the cache of entry {e.cache_from}, whose shape differs")
            if owner.window is not None and (mine.window is None or mine.window > owner.window):
                raise ValueError(f"schedule[{i}] reads further back than entry {e.cache_from} keeps (window {owner.window})")
            entry_group[i] = entry_group[e.cache_from]
    return groups, entry_group


class CacheStorage:
    def __init__(self, schedule, mixers, page_size: int, num_pages, max_requests: int, dtype: torch.dtype, device):
        self.groups, self.entry_group = plan_groups(schedule, mixers)
        counts = [num_pages] * len(self.groups) if isinstance(num_pages, int) else list(num_pages)
        self.manager = CacheManager(self.groups, page_size, counts, max_requests) if self.groups else \
            CacheManager([], page_size, [], max_requests)
        self.page_size, self.dtype, self.device = page_size, dtype, device
        # One page more than the manager hands out, at the end of every cache tensor: the scratch page, which rows
        # that stand for nobody (padding of a captured decode step's batch) write to and read back.
        self.scratch_pages = list(counts)
        # ... and one state slot more than the manager hands out, for the same rows: what they leave there is read by nobody.
        self.scratch_state_slot = max_requests
        self._caches: Dict[int, LayerCache] = {}
        self._states: Dict[int, torch.Tensor] = {}
        for i, e in enumerate(schedule):
            m = mixers[i]
            spec = m.cache_spec()
            if spec is not None and e.cache_from is None:
                g = self.entry_group[i]
                n = counts[g]
                k = torch.zeros((n + 1, spec.n_kv_heads, page_size, spec.k_dim), dtype=dtype, device=device)
                v = torch.zeros((n + 1, spec.n_kv_heads, spec.v_dim, page_size), dtype=dtype, device=device)
                self._caches[i] = LayerCache(k, v, g, page_size)
            st = m.state_spec()
            if st is not None:
                self._states[i] = torch.zeros((max_requests + 1, *st.shape), dtype=_STATE_DTYPES[st.dtype], device=device)
        if self._states:
            self.manager.on_add = self.reset_state       # every admission path starts a request with zero state
        self._bindings: List[MixerBinding] = []
        for i, e in enumerate(schedule):
            owner = i if e.cache_from is None else e.cache_from
            self._bindings.append(MixerBinding(cache=self._caches.get(owner), writes_cache=e.cache_from is None,
                                               state=self._states.get(i)))

    def binding(self, entry: int) -> MixerBinding:
        return self._bindings[entry]

    @property
    def has_state(self) -> bool:
        """Whether any mixer keeps per-request state besides keys and values (a step over it cannot be run twice)."""
        return bool(self._states)

    def reset_state(self, slot: int) -> None:
        """Zero every mixer's state of one slot: a request that starts sees no history."""
        for t in self._states.values():
            t[slot].zero_()

    def bytes_per_token(self) -> int:
        return sum((c.k[0].numel() + c.v[0].numel()) * c.k.element_size() // self.page_size for c in self._caches.values())
