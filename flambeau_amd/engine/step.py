"""The step function: one batch of (request, its next tokens) through the model.

A batch may hold portions of prompts beside single decoded tokens, cut anywhere, each request
at most once.  The step runs only the tokens it is given, from the cache earlier steps left,
and returns the logits at the wanted places.  All metadata of a step (token ids, positions,
request of each token, block tables, wanted rows, what parts asked for) goes to the device in
one copy at its start.

The reference's counterpart is ``Session::forward`` / ``forward_mixed`` /
``forward_decode_batched`` over three parallel arrays (crates/forward/src/runtime/mod.rs:185-264,
:471-486), which allows one portion beside decode rows only and uploads positions and
block-table entries layer by layer (crates/forward/src/core/composites/standard_attn.rs:315-329,
:468-478); here any mix is one batch and the upload happens once.
"""
from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np
import torch

from ..cache.manager import CacheError, CacheManager
from ..cache.storage import CacheStorage
from ..parts.base import HostBatch, StepState


@dataclass
class StepEntry:
    request_id: object
    tokens: list
    want: list = field(default_factory=list)   # places among ``tokens`` whose logits are wanted


class StepError(ValueError):
    pass


class ModelRunner:
    """Owns the model, the cache and the step function."""

    def __init__(self, model, *, n_pages: int, page_size: int, max_slots: int, max_seq_len: int | None = None,
                 max_logit_rows: int | None = None):
        self.model = model
        self.rt = model.rt
        spec = model.spec
        self.max_seq_len = min(max_seq_len or spec.max_position, spec.max_position)
        specs, shares = model.cache_entries()
        self.storage = CacheStorage(specs, shares, self.rt.device, self.rt.dtype, n_pages, page_size, max_slots)
        self.manager = CacheManager(self.storage.group_specs, n_pages, page_size, max_slots, self.max_seq_len)
        self.max_logit_rows = max_logit_rows or self.rt.max_batch_tokens
        self._mixer_classes = model.mixer_classes()
        self._meta_capacity = 0
        self._meta_host = None
        self._meta_dev = None
        self._meta_copied = None     # event: the last metadata copy has left the pinned buffer

    # ------------------------------------------------------------ requests
    def begin(self, request_id) -> bool:
        """Claim a slot for a new request.  False when no slot is free."""
        return self.manager.admit(request_id) is not None

    def end(self, request_id) -> None:
        self.manager.release(request_id)

    def cached_tokens(self, request_id) -> int:
        return self.manager.live[request_id].n_cached

    # ------------------------------------------------------------ metadata
    def _meta_buffers(self, n_ints: int):
        if n_ints > self._meta_capacity:
            cap = max(4096, 1 << (n_ints - 1).bit_length())
            self._meta_host = torch.empty(cap, dtype=torch.int32, pin_memory=True)
            self._meta_dev = torch.empty(cap, dtype=torch.int32, device=self.rt.device)
            self._meta_capacity = cap
        return self._meta_host, self._meta_dev

    def build_step(self, entries, table_width: int | None = None) -> StepState:
        """Validate the entries, reserve their pages and put the batch's metadata on the device."""
        mgr = self.manager
        V = self.model.spec.vocab_size
        seen = set()
        n = 0
        for e in entries:
            if e.request_id in seen:
                raise StepError(f"request {e.request_id!r} appears twice in one step")
            seen.add(e.request_id)
            if e.request_id not in mgr.live:
                raise StepError(f"request {e.request_id!r} is not live (begin it first)")
            if len(e.tokens) == 0:
                raise StepError(f"request {e.request_id!r} brings no tokens")
            for w in e.want:
                if not 0 <= w < len(e.tokens):
                    raise StepError(f"request {e.request_id!r}: wanted place {w} of {len(e.tokens)} tokens")
            n += len(e.tokens)
        if n > self.rt.max_batch_tokens:
            raise StepError(f"{n} tokens in one step, the engine was sized for {self.rt.max_batch_tokens}")
        n_rows = sum(len(e.want) for e in entries)
        if n_rows > self.max_logit_rows:
            raise StepError(f"logits wanted at {n_rows} places, at most {self.max_logit_rows} per step")
        if not mgr.can_cover((e.request_id, mgr.live[e.request_id].n_cached + len(e.tokens)) for e in entries):
            raise CacheError("not enough free pages (or a request beyond the maximum length) for this step")

        tokens = np.empty(n, dtype=np.int32)
        positions = np.empty(n, dtype=np.int32)
        tok_seq = np.empty(n, dtype=np.int32)
        S = len(entries)
        q_starts, q_lens, starts, slots, rows = [], [], [], [], []
        at = 0
        for s, e in enumerate(entries):
            rc = mgr.live[e.request_id]
            k = len(e.tokens)
            mgr.ensure(e.request_id, rc.n_cached + k)
            tokens[at:at + k] = e.tokens
            positions[at:at + k] = np.arange(rc.n_cached, rc.n_cached + k, dtype=np.int32)
            tok_seq[at:at + k] = s
            q_starts.append(at)
            q_lens.append(k)
            starts.append(rc.n_cached)
            slots.append(rc.slot)
            rows += [at + w for w in e.want]
            at += k
        if n and (tokens.min() < 0 or tokens.max() >= V):
            bad = int(tokens[(tokens < 0) | (tokens >= V)][0])
            raise StepError(f"token id {bad} is outside the vocabulary of {V}")
        batch = HostBatch(q_starts, q_lens, starts, slots, n, len(rows))

        need_blocks = max((-(-(st + q) // mgr.page_size) for st, q in zip(starts, q_lens)), default=1)
        width = table_width or max(8, -(-need_blocks // 8) * 8)
        tables = []
        for g in range(len(mgr.groups)):
            t = np.full((S, width), -1, dtype=np.int32)
            for s, e in enumerate(entries):
                row = mgr.table_row(e.request_id, g)
                t[s, :len(row)] = row
            tables.append(t)

        parts = [("tokens", tokens), ("positions", positions), ("tok_seq", tok_seq),
                 ("seq_slots", np.asarray(slots, dtype=np.int32)),
                 ("seq_q_start", np.asarray(q_starts, dtype=np.int32)),
                 ("seq_q_len", np.asarray(q_lens, dtype=np.int32)),
                 ("seq_ctx_len", np.asarray([st + q for st, q in zip(starts, q_lens)], dtype=np.int32)),
                 ("logit_rows", np.asarray(rows, dtype=np.int32))]
        parts += [(f"table{g}", t) for g, t in enumerate(tables)]
        extra_names = []
        for cls in self._mixer_classes:
            for name, arr in cls.step_metadata(batch).items():
                parts.append(("extra:" + name, np.ascontiguousarray(arr, dtype=np.int32)))
                extra_names.append(name)
        dev = self._upload(parts)
        return StepState(
            n_tokens=n, n_seqs=S, tokens=dev["tokens"], positions=dev["positions"], tok_seq=dev["tok_seq"],
            seq_slots=dev["seq_slots"], seq_q_start=dev["seq_q_start"], seq_q_len=dev["seq_q_len"],
            seq_ctx_len=dev["seq_ctx_len"], block_tables=[dev[f"table{g}"] for g in range(len(tables))],
            logit_rows=dev["logit_rows"], host=batch, extra={k: dev["extra:" + k] for k in extra_names})

    def _upload(self, parts) -> dict:
        """One host-to-device copy for all integer arrays; returns device views by name."""
        offsets, total = [], 0
        for _, arr in parts:
            offsets.append(total)
            total += -(-arr.size // 4) * 4 if arr.size else 0   # 16-byte alignment of every array
        if self._meta_copied is not None:
            self._meta_copied.synchronize()
        host, dev = self._meta_buffers(max(total, 1))
        hnp = host.numpy()
        for (name, arr), off in zip(parts, offsets):
            if arr.size:
                hnp[off:off + arr.size] = arr.reshape(-1)
        if total:
            dev[:total].copy_(host[:total], non_blocking=True)
            if self._meta_copied is None:
                self._meta_copied = torch.cuda.Event()
            self._meta_copied.record()
        out = {}
        for (name, arr), off in zip(parts, offsets):
            out[name] = dev[off:off + arr.size].view(arr.shape)
        return out

    # ------------------------------------------------------------ the step
    def step(self, entries):
        """Run one batch.  Returns float32 logits ``[wanted, vocab]`` on the device (rows in the
        order of the entries and of their ``want``), or ``None`` if nothing was wanted.
        The returned tensor is a view of a buffer the next step overwrites."""
        entries = [e if isinstance(e, StepEntry) else StepEntry(*e) for e in entries]
        if not entries:
            return None
        step = self.build_step(entries)
        self.storage.zero_slots(self.manager.take_fresh_slots())
        logits = self.model.forward(step, self.storage.entries, self.max_logit_rows)
        for e in entries:
            self.manager.advance(e.request_id, len(e.tokens))
        return logits
