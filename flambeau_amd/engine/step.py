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

from collections import OrderedDict
from dataclasses import dataclass, field

import numpy as np
import torch

from ..cache.manager import CacheError, CacheManager
from ..cache.storage import CacheStorage
from ..kernels import ops
from ..kernels.library import Program
from ..parts.base import HostBatch, StepState


@dataclass
class StepEntry:
    request_id: object
    tokens: list
    want: list = field(default_factory=list)   # places among ``tokens`` whose logits are wanted
    from_device: int | None = None            # a single token that is still on the device: its row in
                                              # the runner's ``token_feedback`` buffer (``tokens`` is ignored)


class StepError(ValueError):
    pass


class ModelRunner:
    """Owns the model, the cache and the step function."""

    def __init__(self, model, *, n_pages: int, page_size: int, max_slots: int, max_seq_len: int | None = None,
                 max_logit_rows: int | None = None, decode_graphs: bool = True, max_graph_batch: int = 256,
                 step_programs: bool = True, max_programs: int = 96):
        self.model = model
        self.rt = model.rt
        spec = model.spec
        self.max_seq_len = min(max_seq_len or spec.max_position, spec.max_position)
        specs, shares = model.cache_entries()
        self.storage = CacheStorage(specs, shares, self.rt.device, self.rt.dtype, n_pages, page_size, max_slots)
        self.manager = CacheManager(self.storage.group_specs, n_pages, page_size, max_slots, self.max_seq_len)
        self.max_logit_rows = max_logit_rows or self.rt.max_batch_tokens
        self._mixer_classes = model.mixer_classes()
        by_class = getattr(model, "mixers_by_class", lambda: {})()
        self._mixers_of = {c: by_class.get(c, []) for c in self._mixer_classes}
        self._meta_capacity = 0
        self._meta_host = None
        self._meta_dev = None
        self._meta_copied = None     # event: the last metadata copy has left the pinned buffer
        # steps of single tokens replay a captured graph per batch-size bucket, if every mixer
        # of the model says that running a step twice leaves the same cache (graph_safe) and every part
        # of it can be captured (a part that is not replayable may call what a capture does not allow); a
        # model that cannot have its steps of single tokens recorded instead, and the recorded stretches
        # around the blocks in question become graphs of their own
        self.decode_graphs = (bool(decode_graphs) and all(getattr(c, "graph_safe", False) for c in self._mixer_classes)
                              and getattr(model, "capturable", lambda: True)())
        self.max_graph_batch = min(max_graph_batch, max_slots)
        self._graphs: dict[int, "_GraphedStep"] = {}
        # ids drawn on the device in the step before (the sampler's output buffer); entries with
        # ``from_device`` read their token from it, so a step can be enqueued before the host has
        # seen the step before
        self.token_feedback = None
        # Steps that no graph takes (anything with a prompt portion) are recorded while they run and
        # replayed from native code when a step of the same shape and the same kernel choices comes
        # again: ``{key: _RecordedStep}``, least recently used first.
        self.step_programs = bool(step_programs) and model.replayable()
        self.max_programs = max_programs
        self.graph_after_hits = 3           # replays after which a recorded step is turned into a graph
        self._programs: OrderedDict = OrderedDict()
        self.n_replayed = 0
        self.n_recorded = 0

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

    def _validate(self, entries):
        mgr = self.manager
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
        V = self.model.spec.vocab_size
        for e in entries:
            if e.from_device is not None:
                if len(e.tokens) != 1 or self.token_feedback is None or not 0 <= e.from_device < self.token_feedback.shape[0]:
                    raise StepError(f"request {e.request_id!r}: a token from the device needs one place and a feedback buffer")
                continue
            if min(e.tokens) < 0 or max(e.tokens) >= V:
                bad = next(t for t in e.tokens if not 0 <= t < V)
                raise StepError(f"token id {bad} is outside the vocabulary of {V}")
        if not mgr.can_cover((e.request_id, mgr.live[e.request_id].n_cached + len(e.tokens)) for e in entries):
            raise CacheError("not enough free pages (or a request beyond the maximum length) for this step")
        return n

    def _assemble(self, entries, pad_to: int | None = None):
        """Reserve the entries' pages and lay out the batch's metadata as integer arrays.
        ``pad_to``: fixed number of single-token requests (graph replay); the padding rows have
        no pages, write nothing and are never read."""
        mgr = self.manager
        n = sum(len(e.tokens) for e in entries)
        S = len(entries)
        n_pad = (pad_to - S) if pad_to is not None else 0
        tokens = np.zeros(n + n_pad, dtype=np.int32)
        positions = np.zeros(n + n_pad, dtype=np.int32)
        tok_seq = np.empty(n + n_pad, dtype=np.int32)
        token_src = np.full(n + n_pad, -1, dtype=np.int32)
        q_starts, q_lens, starts, slots, rows = [], [], [], [], []
        at = 0
        for s, e in enumerate(entries):
            rc = mgr.live[e.request_id]
            k = len(e.tokens)
            mgr.ensure(e.request_id, rc.n_cached + k)
            if e.from_device is not None:
                token_src[at] = e.from_device
            else:
                tokens[at:at + k] = e.tokens
            positions[at:at + k] = np.arange(rc.n_cached, rc.n_cached + k, dtype=np.int32)
            tok_seq[at:at + k] = s
            q_starts.append(at)
            q_lens.append(k)
            starts.append(rc.n_cached)
            slots.append(rc.slot)
            rows += [at + w for w in e.want]
            at += k
        for s in range(S, S + n_pad):
            tok_seq[at] = s
            q_starts.append(at)
            q_lens.append(1)
            starts.append(0)
            slots.append(0)
            at += 1
        if pad_to is not None:
            rows = list(range(pad_to))          # a fixed-shape step computes every row's logits
        batch = HostBatch(q_starts, q_lens, starts, slots, n + n_pad, len(rows),
                          ctx_bound=self.max_seq_len if pad_to is not None else None,
                          every_row=rows == list(range(n + n_pad)))
        if pad_to is not None:
            width = mgr.max_blocks
        else:
            # the tables' width is a power of two: it is part of a step's shape (recorded steps are
            # keyed by it) and should not change with every page a request gains
            need_blocks = max((-(-(st + q) // mgr.page_size) for st, q in zip(starts, q_lens)), default=1)
            width = max(8, 1 << (need_blocks - 1).bit_length())
        tables = []
        for g in range(len(mgr.groups)):
            t = np.full((S + n_pad, width), -1, dtype=np.int32)
            for s, e in enumerate(entries):
                row = mgr.table_row(e.request_id, g)
                t[s, :len(row)] = row
            tables.append(t)
        parts = [("tokens", tokens), ("token_src", token_src), ("positions", positions), ("tok_seq", tok_seq),
                 ("seq_slots", np.asarray(slots, dtype=np.int32)),
                 ("seq_q_start", np.asarray(q_starts, dtype=np.int32)),
                 ("seq_q_len", np.asarray(q_lens, dtype=np.int32)),
                 ("seq_ctx_len", np.asarray([st + q for st, q in zip(starts, q_lens)], dtype=np.int32)),
                 ("logit_rows", np.asarray(rows, dtype=np.int32))]
        parts += [(f"table{g}", t) for g, t in enumerate(tables)]
        for cls in self._mixer_classes:
            # (a class that wants to see its mixers, for their sizes, has step_metadata_for)
            wanted = (cls.step_metadata_for(batch, self._mixers_of[cls]) if hasattr(cls, "step_metadata_for")
                      else cls.step_metadata(batch))
            for name, arr in wanted.items():
                parts.append(("extra:" + name, np.ascontiguousarray(arr, dtype=np.int32)))
        return batch, parts

    def _feed(self, dev, needed: bool) -> None:
        """Fill in the tokens that are still on the device."""
        if needed:
            ops.feed_tokens(dev["tokens"], self.token_feedback, dev["token_src"])

    def _state_from(self, batch, parts, dev) -> StepState:
        extra = {name[6:]: dev[name] for name, _ in parts if name.startswith("extra:")}
        n_groups = len(self.manager.groups)
        return StepState(
            n_tokens=batch.n_tokens, n_seqs=batch.n_seqs, tokens=dev["tokens"], positions=dev["positions"],
            tok_seq=dev["tok_seq"], seq_slots=dev["seq_slots"], seq_q_start=dev["seq_q_start"],
            seq_q_len=dev["seq_q_len"], seq_ctx_len=dev["seq_ctx_len"],
            block_tables=[dev[f"table{g}"] for g in range(n_groups)], logit_rows=dev["logit_rows"],
            host=batch, extra=extra)

    def build_step(self, entries) -> StepState:
        """Validate the entries, reserve their pages and put the batch's metadata on the device."""
        self._validate(entries)
        batch, parts = self._assemble(entries)
        return self._state_from(batch, parts, self._upload(parts))

    @staticmethod
    def _layout(parts):
        offsets, total = [], 0
        for _, arr in parts:
            offsets.append(total)
            total += -(-arr.size // 4) * 4 if arr.size else 0   # 16-byte alignment of every array
        return offsets, total

    def _upload(self, parts, dev=None) -> dict:
        """One host-to-device copy for all integer arrays; returns device views by name.
        ``dev``: a fixed device buffer (a captured graph's own) instead of the shared one."""
        offsets, total = self._layout(parts)
        if self._meta_copied is not None:
            self._meta_copied.synchronize()
        host, shared = self._meta_buffers(max(total, 1))
        if dev is None:
            dev = shared
        elif dev.numel() < total:
            raise StepError("metadata of a fixed-shape step outgrew its buffer")
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
        self._validate(entries)
        fresh = self.manager.take_fresh_slots()
        self.storage.zero_slots(fresh)
        if self.decode_graphs and self._bucket(len(entries)) <= min(self.max_graph_batch, self.rt.max_batch_tokens) \
                and len(entries) <= self.max_graph_batch and all(len(e.tokens) == 1 for e in entries):
            logits = self._step_graphed(entries)
        else:
            batch, parts = self._assemble(entries)
            dev = self._upload(parts)
            feed = any(e.from_device is not None for e in entries)
            if self.step_programs:
                logits = self._step_recorded(batch, parts, dev, feed)
            else:
                self._feed(dev, feed)
                logits = self.model.forward(self._state_from(batch, parts, dev), self.storage.entries, self.max_logit_rows)
        for e in entries:
            self.manager.advance(e.request_id, len(e.tokens))
        return logits

    # ------------------------------------------------------------ recorded steps
    def _program_key(self, batch, parts, feed: bool):
        """Everything that decides which kernels a step launches and with which arguments: rows per
        request, number and pattern of the wanted rows, shapes of all metadata (they fix where each
        array lies on the device), whether tokens come from the device, and what the mixers decide
        from the contexts' lengths."""
        return (tuple(batch.q_lens), batch.n_logit_rows, batch.every_row, feed,
                tuple(arr.shape for _, arr in parts), self.model.step_signature(batch))

    def _step_recorded(self, batch, parts, dev, feed: bool):
        key = self._program_key(batch, parts, feed)
        hit = self._programs.get(key)
        valid = (self.rt.generation, self._meta_dev.data_ptr())
        stream = torch.cuda.current_stream().cuda_stream
        if hit is not None and hit.valid == valid:
            self._programs.move_to_end(key)
            hit.hits += 1
            if hit.hits >= self.graph_after_hits and not hit.graphs:
                # a shape that keeps coming back: the launches of every recorded stretch become a graph
                # (they are this library's kernels only, with fixed arguments), which costs one launch to
                # replay; blocks that cannot be recorded still run as they are between the graphs
                for i, s in enumerate(hit.stretches):
                    if isinstance(s, Program):
                        graph = torch.cuda.CUDAGraph()
                        with torch.cuda.graph(graph):
                            s.run(torch.cuda.current_stream().cuda_stream)
                        hit.graphs[i] = graph
            if len(hit.stretches) == 1 and isinstance(hit.stretches[0], Program):
                if hit.graphs:
                    hit.graphs[0].replay()
                else:
                    hit.stretches[0].run(stream)
            else:
                now = self._state_from(batch, parts, dev)
                with ops.pinned_stream():
                    for i, s in enumerate(hit.stretches):
                        if i in hit.graphs:
                            hit.graphs[i].replay()
                        elif isinstance(s, Program):
                            s.run(stream)
                        else:
                            s(now)
            self.n_replayed += 1
            return hit.logits
        recorder = _StepRecorder()
        state = self._state_from(batch, parts, dev)
        state.recorder = recorder
        with recorder:
            self._feed(dev, feed)
            logits = self.model.forward(state, self.storage.entries, self.max_logit_rows)
        state.recorder = None
        # (a buffer that grew during this very step moved before it was used: the generation is read afterwards)
        self._programs[key] = _RecordedStep(recorder.stretches, logits, (self.rt.generation, self._meta_dev.data_ptr()))
        self._programs.move_to_end(key)
        while len(self._programs) > self.max_programs:
            self._programs.popitem(last=False)
        self.n_recorded += 1
        return logits

    # ------------------------------------------------------------ captured decode steps
    def _bucket(self, n: int) -> int:
        b = 1
        while b < n:
            b *= 2
        return b if b <= self.max_graph_batch else max(n, self.max_graph_batch)

    def _step_graphed(self, entries):
        """A step of single tokens: pad to the bucket's size, copy the metadata into the graph's
        own buffer, replay.  The first step of a bucket runs eagerly once (buffers are made),
        is captured, and replayed; a step leaves the same cache however often it runs."""
        bk = self._bucket(len(entries))
        batch, parts = self._assemble(entries, pad_to=bk)
        # one graph per bucket and per thing the mixers decide from the contexts (whether a kernel that
        # merges splits of the keys runs at all, for one); the graphs of a bucket share their buffers
        key = (bk, self.model.step_signature(batch))
        gs = self._graphs.get(key)
        if gs is None:
            _, total = self._layout(parts)
            gs = _GraphedStep(torch.empty(max(total, 1), dtype=torch.int32, device=self.rt.device))
            self._graphs[key] = gs
        dev = self._upload(parts, gs.meta)
        feedback = self.token_feedback is not None
        if gs.graph is None:
            step = self._state_from(batch, parts, dev)
            with self.rt.scope(f"graph{bk}"):
                self._feed(dev, feedback)
                self.model.forward(step, self.storage.entries, bk)          # makes the buffers
                torch.cuda.current_stream().synchronize()
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph):
                    self._feed(dev, feedback)          # part of the graph: a no-op when no token comes from the device
                    gs.logits = self.model.forward(step, self.storage.entries, bk)
            gs.graph = graph
            gs.feedback = feedback
        elif gs.feedback != feedback:
            raise StepError("the token feedback buffer must be set before the first captured step")
        gs.graph.replay()
        wanted = [i for i, e in enumerate(entries) for _ in e.want]     # one row per wanted place
        if not wanted:
            return None
        if wanted == list(range(len(wanted))):
            return gs.logits[:len(wanted)]
        return gs.logits[torch.tensor(wanted, device=self.rt.device)]


class _StepRecorder:
    """Records a step as stretches of launches (``Program``) with, between them, whatever a model
    says cannot be recorded (``cut``): callables that take the step's state and run again at every
    replay."""

    def __init__(self):
        self.stretches: list = []
        self._open = None

    def _begin(self):
        self._open = Program()
        self._ctx = self._open.recording()
        self._ctx.__enter__()

    def _end(self):
        self._ctx.__exit__(None, None, None)
        if len(self._open):
            self.stretches.append(self._open)
        self._open = None

    def __enter__(self):
        self._begin()
        return self

    def __exit__(self, *exc):
        self._end()

    def cut(self, run_again) -> None:
        """End the stretch that is being recorded, note ``run_again(step_state)`` for the replays,
        begin the next stretch.  The caller runs the thing itself now, with recording suspended."""
        self._end()
        self.stretches.append(run_again)
        self._begin()


class _RecordedStep:
    def __init__(self, stretches, logits, valid):
        self.stretches = stretches  # Programs, and callables for what cannot be recorded
        self.logits = logits
        self.valid = valid          # (buffer generation, address of the metadata) the arguments belong to
        self.hits = 0
        self.graphs = {}            # index of a stretch -> the device graph of its launches


class _GraphedStep:
    def __init__(self, meta):
        self.meta = meta
        self.graph = None
        self.logits = None
        self.feedback = False
