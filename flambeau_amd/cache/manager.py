"""The cache manager: pages, block tables, windows, state slots.  Host-side bookkeeping only.

Keys and values live in pages of ``page_size`` tokens.  Layers whose caches have the
same shape and window form a *group*; a group has one free list and, for each live
request, one block table (entry ``i`` = page holding tokens ``[i*ps, (i+1)*ps)``) that
serves all its layers.  Pages return to the free list when a request ends, when it is
pre-empted, and, in a windowed group, as soon as every token in them lies below the
window of all future queries; the table keeps a hole (-1) there so that token ``t`` is
always found at ``table[t // ps]``.

Beside the pages every live request holds one *slot*: the index of its record in the
per-request state of fixed size that layers may keep (none for attention).

The reference's counterpart: ``PagePool`` with a FIFO free list and per-slot held pages,
one per layer (crates/forward/src/core/scratch.rs:602-703), block tables of
``ceil(max_seq_len / page_size)`` entries (:438-463), release only at request end
(crates/server/src/routes.rs:544-547), an error when pages run out
(crates/forward/src/core/composites/standard_attn.rs:449-458).  Here the scheduler asks
``can_cover`` before it builds a batch, so a step never fails for want of a page.
"""
from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field


class CacheError(RuntimeError):
    pass


class PagePool:
    """Free list of one group.  FIFO, as the reference's (scratch.rs:602-640)."""

    def __init__(self, n_pages: int):
        if n_pages < 1:
            raise CacheError(f"a page pool needs at least one page, got {n_pages}")
        self.n_pages = n_pages
        self._free = deque(range(n_pages))
        self._is_free = [True] * n_pages
        self.n_acquired = 0                     # pages handed out so far (more than n_pages: pages were used again)

    @property
    def n_free(self) -> int:
        return len(self._free)

    def acquire(self) -> int | None:
        if not self._free:
            return None
        p = self._free.popleft()
        self._is_free[p] = False
        self.n_acquired += 1
        return p

    def release(self, page: int) -> None:
        if not 0 <= page < self.n_pages:
            raise CacheError(f"page {page} is not in the pool of {self.n_pages}")
        if self._is_free[page]:
            raise CacheError(f"page {page} freed twice")
        self._is_free[page] = True
        self._free.append(page)


@dataclass(frozen=True)
class GroupSpec:
    """A cache group as the manager sees it: all it reads is ``window`` (newest rows still needed,
    0 = all).  Any object with that attribute serves (``parts.base.PageGroup`` in the engine)."""
    n_kv_heads: int = 1
    head_dim: int = 1
    window: int = 0


@dataclass
class RequestCache:
    """What one live request holds."""
    request_id: object
    slot: int
    n_cached: int = 0                                  # tokens whose keys are in the cache
    tables: list = field(default_factory=list)         # per group: list of page ids, -1 = released
    first_live: list = field(default_factory=list)     # per group: first block not yet released


class CacheManager:
    def __init__(self, groups, n_pages: int, page_size: int, max_slots: int, max_seq_len: int):
        if page_size < 1:
            raise CacheError(f"page size must be positive, got {page_size}")
        self.groups = list(groups)
        self.page_size = page_size
        self.max_slots = max_slots
        self.max_seq_len = max_seq_len
        self.max_blocks = -(-max_seq_len // page_size)
        self.pools = [PagePool(n_pages) for _ in self.groups]
        self._free_slots = deque(range(max_slots))
        self._fresh_slots: list[int] = []
        self.live: dict[object, RequestCache] = {}

    # ------------------------------------------------------------ slots
    @property
    def n_free_slots(self) -> int:
        return len(self._free_slots)

    def admit(self, request_id) -> RequestCache | None:
        """Claim a slot for a new request; ``None`` when all slots are taken."""
        if request_id in self.live:
            raise CacheError(f"request {request_id!r} is already live")
        if not self._free_slots:
            return None
        slot = self._free_slots.popleft()
        rc = RequestCache(request_id, slot, 0, [[] for _ in self.groups], [0 for _ in self.groups])
        self.live[request_id] = rc
        self._fresh_slots.append(slot)
        return rc

    def take_fresh_slots(self) -> list[int]:
        """Slots claimed since the last call: their fixed-size state must be zeroed."""
        out, self._fresh_slots = self._fresh_slots, []
        return out

    # ------------------------------------------------------------ pages
    def _blocks_for(self, n_tokens: int) -> int:
        return -(-n_tokens // self.page_size)

    def pages_needed(self, request_id, upto: int) -> list[int]:
        """New pages per group so that tokens ``[0, upto)`` of the request have a place."""
        rc = self.live[request_id]
        return [max(0, self._blocks_for(upto) - len(t)) for t in rc.tables]

    def can_cover(self, wants) -> bool:
        """``wants``: iterable of (request_id, upto).  True if all fit in the free lists at once."""
        need = [0] * len(self.groups)
        for rid, upto in wants:
            if upto > self.max_seq_len:
                return False
            for g, k in enumerate(self.pages_needed(rid, upto)):
                need[g] += k
        return all(n <= pool.n_free for n, pool in zip(need, self.pools))

    def free_pages(self) -> list[int]:
        return [p.n_free for p in self.pools]

    def ensure(self, request_id, upto: int) -> None:
        """Give the request pages for tokens ``[n_cached, upto)``.  All or nothing."""
        rc = self.live[request_id]
        if upto > self.max_seq_len:
            raise CacheError(f"request {request_id!r}: {upto} tokens exceed the maximum of {self.max_seq_len}")
        need = self.pages_needed(request_id, upto)
        for g, k in enumerate(need):
            if k > self.pools[g].n_free:
                raise CacheError(
                    f"request {request_id!r}: group {g} needs {k} pages, {self.pools[g].n_free} free")
        for g, k in enumerate(need):
            for _ in range(k):
                rc.tables[g].append(self.pools[g].acquire())

    def advance(self, request_id, n_tokens: int) -> None:
        """The request's next ``n_tokens`` are now in the cache.  Pages that fell out of a
        group's window go back to its free list."""
        rc = self.live[request_id]
        new_len = rc.n_cached + n_tokens
        for g, t in enumerate(rc.tables):
            if new_len > len(t) * self.page_size:
                raise CacheError(f"request {request_id!r}: advanced to {new_len} tokens beyond its pages")
        rc.n_cached = new_len
        for g, spec in enumerate(self.groups):
            if spec.window <= 0:
                continue
            # the next query sits at position new_len and sees keys >= new_len - window + 1
            first_needed = new_len - spec.window + 1
            dead_blocks = max(0, first_needed) // self.page_size
            t = rc.tables[g]
            for b in range(rc.first_live[g], min(dead_blocks, len(t))):
                if t[b] >= 0:
                    self.pools[g].release(t[b])
                    t[b] = -1
            rc.first_live[g] = max(rc.first_live[g], min(dead_blocks, len(t)))

    def release(self, request_id) -> None:
        """The request ends (or is pre-empted): all its pages and its slot are given back."""
        rc = self.live.pop(request_id, None)
        if rc is None:
            raise CacheError(f"request {request_id!r} is not live")
        for g, t in enumerate(rc.tables):
            for page in t:
                if page >= 0:
                    self.pools[g].release(page)
        self._free_slots.append(rc.slot)
        if rc.slot in self._fresh_slots:
            self._fresh_slots.remove(rc.slot)

    def table_row(self, request_id, group: int) -> list[int]:
        return self.live[request_id].tables[group]

    # ------------------------------------------------------------ checks
    def check_invariants(self) -> None:
        """No page lost, held twice or both held and free; slots likewise."""
        for g, pool in enumerate(self.pools):
            held = []
            for rc in self.live.values():
                held += [p for p in rc.tables[g] if p >= 0]
            if len(held) != len(set(held)):
                raise CacheError(f"group {g}: a page is held twice")
            free = list(pool._free)
            if len(free) != len(set(free)):
                raise CacheError(f"group {g}: a page is on the free list twice")
            if set(held) & set(free):
                raise CacheError(f"group {g}: a page is both held and free")
            if len(held) + len(free) != pool.n_pages:
                raise CacheError(f"group {g}: {pool.n_pages - len(held) - len(free)} pages lost")
        slots = [rc.slot for rc in self.live.values()]
        if len(slots) != len(set(slots)):
            raise CacheError("a slot is held twice")
        if set(slots) & set(self._free_slots) or len(slots) + len(self._free_slots) != self.max_slots:
            raise CacheError("slots lost or both held and free")
