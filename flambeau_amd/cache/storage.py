"""Device memory of the caches: one pool per group of paged caches, one table of records per cache
that keeps a state per slot.

What a cache looks like is its spec's business (``parts.base.CacheSpec``): the storage asks a spec
which group of pages it belongs to, lets the first spec of a group allocate the group's pool, and
hands every entry its view of it.  For keys and values the pool is ``[entries_in_group, n_pages, 2
(K, V), n_kv_heads, page_size, head_dim]`` in the compute dtype, so that one (page, kv head) holds
``page_size`` rows of ``head_dim`` values back to back: a decode kernel streams whole pages of one
head.  (The reference keeps ``[n_pages, page_size, kv_width]`` per layer,
crates/forward/src/core/scratch.rs:453-586.)
"""
from __future__ import annotations

import torch

from ..parts.base import CacheSpec, LayerCache


class CacheStorage:
    def __init__(self, entry_specs, shares, device, dtype, n_pages: int, page_size: int, max_slots: int):
        """``entry_specs[i]``: cache spec of run-order entry ``i`` (or None);
        ``shares[i]``: index of the earlier entry whose cache entry ``i`` reads instead of
        having its own (or None)."""
        self.page_size = page_size
        self.n_pages = n_pages
        for i, spec in enumerate(entry_specs):
            if spec is not None and not isinstance(spec, CacheSpec):
                raise TypeError(f"run-order entry {i}: {spec!r} is no cache spec")
        self.group_specs: list = []               # page groups (each has a ``window``), in order of first use
        self._group_makers: list = []             # the spec that allocates each group's pool
        members: list[list[int]] = []
        owner_group: dict[int, int] = {}
        for i, (spec, share) in enumerate(zip(entry_specs, shares)):
            group = spec.page_group() if spec is not None and share is None else None
            if group is None:
                continue
            if group not in self.group_specs:
                self.group_specs.append(group)
                self._group_makers.append(spec)
                members.append([])
            g = self.group_specs.index(group)
            members[g].append(i)
            owner_group[i] = g
        self.pools = [maker.allocate_pool(len(m), n_pages, page_size, dtype, device)
                      for maker, m in zip(self._group_makers, members)]
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
            if spec is not None:
                if spec.page_group() is not None:
                    g = owner_group[src]
                    lc.group = g
                    lc.kv = spec.layer_view(self.pools[g], members[g].index(src))
                if src not in self.states:
                    state = spec.allocate_state(max_slots, device)
                    if state is not None:
                        self.states[src] = state
                lc.state = self.states.get(src)
            self.entries.append(lc)
        self._bytes_per_token = sum(spec.bytes_per_token(torch.empty((), dtype=dtype).element_size())
                                    for spec, share in zip(entry_specs, shares) if spec is not None and share is None)

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
        return self._bytes_per_token

    def nbytes(self) -> int:
        return sum(p.numel() * p.element_size() for p in self.pools) + sum(
            t.numel() * t.element_size() for t in self.states.values())
