"""Sampling on the device: argmax, the temperature draw, and the draw through top-k, top-p and
min-p.

The host supplies one uniform number per row from the request's own generator, so a
request's tokens do not depend on what else is in the batch; the kernels do the softmax, the
selection and the inverse-CDF walk.  (The reference has a device sampler too, a single-block
top-k softmax, crates/kernels-hip/src/kernels/sampler_topk_softmax_f32.cu, and keeps the walk
on the host.)  Penalties and a logit bias need the request's history and stay on the host."""
from __future__ import annotations

import torch

from ..kernels import ops


class DeviceSampler:
    def __init__(self, device, max_rows: int):
        self.device = device
        self.max_rows = max_rows
        # per row: 1 / temperature, the uniform number, top-k (0: none), top-p (0: none), min-p (0: none)
        self._host = torch.zeros((2, 5, max_rows), dtype=torch.float32, pin_memory=True)
        self._dev = torch.zeros((5, max_rows), dtype=torch.float32, device=device)
        self.ids = torch.empty(max_rows, dtype=torch.int32, device=device)     # the last draw, on the device
        self._ids_host = torch.empty((2, max_rows), dtype=torch.int32, pin_memory=True)
        self._events = [torch.cuda.Event(), torch.cuda.Event()]
        self._turn = 0
        self._stash = None           # scratch of the filtered draw for vocabularies beyond 32,768

    def sample_async(self, logits, inv_temps, uniforms, filters=None):
        """Enqueue the draw for ``logits`` float32 [R, V] (per row ``inv_temp``, <= 0: argmax, and a
        uniform number in [0, 1); ``filters``: per row ``(top_k, top_p, min_p)`` with ``None`` or 0 for
        what is not asked for).  The ids stay in ``self.ids`` for the next step and are copied to
        the host asynchronously; returns a handle for ``collect``."""
        R = logits.shape[0]
        if R > self.max_rows:
            raise ValueError(f"{R} rows to sample, sampler sized for {self.max_rows}")
        k = self._turn
        self._turn ^= 1
        self._events[k].synchronize()           # the host buffers of this turn are free again
        ids = self.ids[:R]
        if R:
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
            self._ids_host[k, :R].copy_(ids, non_blocking=True)
        self._events[k].record()
        return k, R

    def collect(self, handle) -> list:
        k, R = handle
        self._events[k].synchronize()
        return self._ids_host[k, :R].tolist()

    def sample(self, logits, inv_temps, uniforms, filters=None) -> list:
        return self.collect(self.sample_async(logits, inv_temps, uniforms, filters))
