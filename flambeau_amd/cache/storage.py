"""Device memory of the caches: one pool per group of layers, one state table per stateful layer.

Layout of a group's pool: ``[entries_in_group, n_pages, 2 (K, V), n_kv_heads, page_size,
head_dim]`` in the compute dtype, so that one (page, kv head) holds ``page_size`` rows of
``head_dim`` values back to back: a decode kernel streams whole pages of one head.
(The reference keeps ``[n_pages, page_size, kv_width]`` per layer,
crates/forward/src/core/scratch.rs:453-586.)
"""
from __future__ import annotations

import torch

from ..kernels.ops import PagedLayerCache
from ..parts.base import LayerCache, PagedKVSpec, StateSpec
from .manager import GroupSpec


class CacheStorage:
    def __init__(self, entry_specs, shares, device, dtype, n_pages: int, page_size: int, max_slots: int):
        """``entry_specs[i]``: cache spec of run-order entry ``i`` (or None);
        ``shares[i]``: index of the earlier entry whose cache entry ``i`` reads instead of
        having its own (or None)."""
        self.page_size = page_size
        self.n_pages = n_pages
        self.group_specs: list[GroupSpec] = []
        members: list[list[int]] = []
        owner_group: dict[int, int] = {}
        for i, (spec, share) in enumerate(zip(entry_specs, shares)):
            if share is not None or not isinstance(spec, PagedKVSpec):
                continue
            gs = GroupSpec(spec.n_kv_heads, spec.head_dim, spec.window)
            if gs not in self.group_specs:
                self.group_specs.append(gs)
                members.append([])
            g = self.group_specs.index(gs)
            members[g].append(i)
            owner_group[i] = g
        self.pools = [
            torch.zeros((len(m), n_pages, 2, gs.n_kv_heads, page_size, gs.head_dim), dtype=dtype, device=device)
            for gs, m in zip(self.group_specs, members)
        ]
        self.states: dict[int, torch.Tensor] = {}
        self.entries: list[LayerCache] = []
        for i, (spec, share) in enumerate(zip(entry_specs, shares)):
            src = i if share is None else share
            if share is not None:
                if not 0 <= share < i or shares[share] is not None:
                    raise ValueError(f"run-order entry {i} may only read the cache of an earlier entry that owns one")
                if entry_specs[share] != spec:
                    raise ValueError(f"run-order entry {i} reads the cache of entry {share}, whose shape differs")
            lc = LayerCache(writes=share is None)
            if isinstance(spec, PagedKVSpec):
                g = owner_group[src]
                lc.group = g
                lc.kv = PagedLayerCache(self.pools[g][members[g].index(src)])
            elif isinstance(spec, StateSpec):
                if src not in self.states:
                    self.states[src] = torch.zeros((max_slots, *spec.shape), dtype=spec.dtype, device=device)
                lc.state = self.states[src]
            elif spec is not None:
                raise TypeError(f"run-order entry {i}: unknown cache spec {spec!r}")
            self.entries.append(lc)

    def zero_slots(self, slots) -> None:
        """Fixed-size state starts at zero for a newly claimed slot
        (crates/forward/src/core/scratch.rs:1530-1572 does the same per slot)."""
        if not slots or not self.states:
            return
        idx = torch.tensor(list(slots), dtype=torch.long, device=next(iter(self.states.values())).device)
        for t in self.states.values():
            t.index_fill_(0, idx, 0)

    def fill(self, value: float) -> None:
        """Overwrite every page of every pool (a debugging aid: with NaN, a read of a row that was
        never written, or of a stale one that should have been masked, shows in the logits)."""
        for p in self.pools:
            p.fill_(value)

    def bytes_per_token(self) -> int:
        return sum(p.shape[0] * 2 * p.shape[3] * p.shape[5] * p.element_size() for p in self.pools)

    def nbytes(self) -> int:
        return sum(p.numel() * p.element_size() for p in self.pools) + sum(
            t.numel() * t.element_size() for t in self.states.values())
