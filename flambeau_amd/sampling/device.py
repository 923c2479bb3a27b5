"""Sampling on the device: argmax, the temperature draw, and the draw through top-k, top-p and
min-p.

The host supplies one uniform number per row from the request's own generator, so a
request's tokens do not depend on what else is in the batch; the kernels do the softmax, the
selection and the inverse-CDF walk.  (The reference has a device sampler too, a single-block
top-k softmax, crates/kernels-hip/src/kernels/sampler_topk_softmax_f32.cu, and keeps the walk
on the host.)  Penalties and a logit bias are applied to the logits on the device before the draw:
the history of generated tokens is a row of counts per request slot that every draw bumps, so
neither the logits nor the history travel."""
from __future__ import annotations

import torch

from ..kernels import ops
from .params import DEVICE_BIAS_MAX as BIAS_MAX


class DeviceSampler:
    def __init__(self, device, max_rows: int, vocab_size: int | None = None):
        """``vocab_size``: if given, the counts for the penalties and the scratch of the filtered draw
        are made now, beside everything else that is sized when an engine is built (64 + 128 MB at 256
        rows and a vocabulary of 131,072); without it they are made when a request first needs them."""
        self.device = device
        self.max_rows = max_rows
        # per row: 1 / temperature, the uniform number, top-k (0: none), top-p (0: none), min-p (0: none),
        # history slot (-1: none), repetition, presence and frequency penalty
        self._host = torch.zeros((2, 9, max_rows), dtype=torch.float32, pin_memory=True)
        self._dev = torch.zeros((9, max_rows), dtype=torch.float32, device=device)
        # logit bias of a step as (row, token, value) triples
        self._bias_host = torch.zeros((2, 3, max_rows * BIAS_MAX), dtype=torch.float32, pin_memory=True)
        self._bias_dev = torch.zeros((3, max_rows * BIAS_MAX), dtype=torch.float32, device=device)
        self._counts = None          # int16 [max_rows, V]: how often a slot's request generated each token
        self._owner = {}             # slot -> (the request whose history the slot's row holds, tokens counted)
        self.ids = torch.empty(max_rows, dtype=torch.int32, device=device)     # the last draw, on the device
        self._ids_host = torch.empty((2, max_rows), dtype=torch.int32, pin_memory=True)
        self._events = [torch.cuda.Event(), torch.cuda.Event()]
        self._turn = 0
        self._stash = None           # scratch of the filtered draw for vocabularies beyond 32,768
        if vocab_size is not None:
            self._counts = torch.zeros((max_rows, vocab_size), dtype=torch.int16, device=device)
            if vocab_size > 32768:
                self._stash = torch.empty(max_rows * vocab_size, dtype=torch.int32, device=device)

    def _histories(self, k, logits, histories):
        """Penalties of the rows that ask for them; returns the device array of their slots."""
        R, V = logits.shape
        if self._counts is None or self._counts.shape[1] != V:
            self._counts = torch.zeros((self.max_rows, V), dtype=torch.int16, device=self.device)
            self._owner = {}
        h = self._host[k].numpy()
        h[5, :R] = -1.0
        for i, hist in enumerate(histories):
            if hist is None:
                continue
            slot, owner, generated, rp, pp, fp = hist
            if not 0 <= slot < self.max_rows:
                raise ValueError(f"history slot {slot}, the sampler has {self.max_rows}")
            if not self.holds_history(slot, owner, len(generated)):
                # the row holds another request's counts, or this request's from before it generated
                # tokens in another slot: count what it has generated so far
                tokens = torch.tensor(list(generated), dtype=torch.int32).to(self.device)
                ops.sample_history(self._counts, slot, tokens)
            self._owner[slot] = (owner, len(generated) + 1)      # this draw joins the row
            h[5, i], h[6, i], h[7, i], h[8, i] = slot, rp, pp, fp
        for a in range(5, 9):
            self._dev[a, :R].copy_(self._host[k, a, :R], non_blocking=True)
        ops.sample_penalise(logits, self._counts, *(self._dev[a, :R] for a in range(5, 9)))
        return self._dev[5, :R]

    def _biases(self, k, logits, biases):
        V = logits.shape[1]
        triples = [(i, int(t), float(b)) for i, bias in enumerate(biases) if bias
                   for t, b in bias.items() if 0 <= int(t) < V]
        n = len(triples)
        if n > self._bias_dev.shape[1]:
            raise ValueError(f"{n} logit-bias entries in a step, the sampler takes {self._bias_dev.shape[1]}")
        if n:
            self._bias_host[k].numpy()[:, :n] = list(zip(*triples))
            for a in range(3):
                self._bias_dev[a, :n].copy_(self._bias_host[k, a, :n], non_blocking=True)
            ops.sample_bias(logits, *(self._bias_dev[a, :n] for a in range(3)))

    def holds_history(self, slot: int, owner, n_generated: int) -> bool:
        """Whether ``slot``'s row of counts holds exactly the ``n_generated`` tokens that ``owner`` has
        generated (else the next draw counts its tokens anew): the row is the request's, and the
        request has drawn every token since in this slot."""
        held = self._owner.get(slot)
        return held is not None and held[0] is owner and held[1] == n_generated

    def sample_async(self, logits, inv_temps, uniforms, filters=None, histories=None, biases=None):
        """Enqueue the draw for ``logits`` float32 [R, V] (per row ``inv_temp``, <= 0: argmax, and a
        uniform number in [0, 1); ``filters``: per row ``(top_k, top_p, min_p)`` with ``None`` or 0 for
        what is not asked for; ``histories``: per row ``None`` or ``(slot, owner, generated, repetition,
        presence, frequency)``, the penalties over the tokens the request ``owner`` has generated, which
        row ``slot`` of the counts follows from draw to draw (``generated`` is read only when the slot
        held another request's); ``biases``: per row ``None`` or ``{token: bias}``.  Penalties and bias
        change ``logits`` in place.  The ids stay in ``self.ids`` for the next step and are copied
        to the host asynchronously; returns a handle for ``collect``."""
        R = logits.shape[0]
        if R > self.max_rows:
            raise ValueError(f"{R} rows to sample, sampler sized for {self.max_rows}")
        k = self._turn
        self._turn ^= 1
        self._events[k].synchronize()           # the host buffers of this turn are free again
        ids = self.ids[:R]
        if R:
            slots = None
            if histories is not None and any(h is not None for h in histories):
                slots = self._histories(k, logits, histories)
            if biases is not None and any(biases):
                self._biases(k, logits, biases)
            if all(t <= 0.0 for t in inv_temps):
                ops.argmax(logits, ids)
            else:
                filtered = filters is not None and any(t > 0.0 and any(f) for t, f in zip(inv_temps, filters))
                h = self._host[k].numpy()
                h[0, :R] = inv_temps
                h[1, :R] = uniforms
                n_arrays = 2
                if filtered:
                    h[2, :R] = [float(f[0] or 0) for f in filters]
                    h[3, :R] = [float(f[1] or 0.0) for f in filters]
                    h[4, :R] = [float(f[2] or 0.0) for f in filters]
                    n_arrays = 5
                for a in range(n_arrays):
                    self._dev[a, :R].copy_(self._host[k, a, :R], non_blocking=True)
                ops.sample(logits, self._dev[0, :R], self._dev[1, :R], ids)
                if filtered:
                    # rows with a filter are drawn again, through it; the others keep their draw
                    V = logits.shape[1]
                    if V > 32768 and (self._stash is None or self._stash.numel() < self.max_rows * V):
                        self._stash = torch.empty(self.max_rows * V, dtype=torch.int32, device=self.device)
                    ops.sample_filtered(logits, self._dev[0, :R], self._dev[1, :R], self._dev[2, :R], self._dev[3, :R],
                                        self._dev[4, :R], ids, stash=self._stash if V > 32768 else None)
            if slots is not None:
                ops.sample_count(self._counts, slots, ids)
            self._ids_host[k, :R].copy_(ids, non_blocking=True)
        self._events[k].record()
        return k, R

    def collect(self, handle) -> list:
        k, R = handle
        self._events[k].synchronize()
        return self._ids_host[k, :R].tolist()

    def sample(self, logits, inv_temps, uniforms, filters=None, histories=None, biases=None) -> list:
        return self.collect(self.sample_async(logits, inv_temps, uniforms, filters, histories, biases))
