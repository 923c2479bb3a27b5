"""Sampling on the device for the common cases: argmax and a plain temperature draw.

The host supplies one uniform number per row from the request's own generator, so a
request's tokens do not depend on what else is in the batch; the kernel does the softmax and
the inverse-CDF walk in index order.  (The reference has a device sampler too, a single-block
top-k softmax, crates/kernels-hip/src/kernels/sampler_topk_softmax_f32.cu, and keeps the walk
on the host.)"""
from __future__ import annotations

import torch

from ..kernels import ops


class DeviceSampler:
    def __init__(self, device, max_rows: int):
        self.device = device
        self.max_rows = max_rows
        self._host = torch.empty((2, 2, max_rows), dtype=torch.float32, pin_memory=True)
        self._dev = torch.empty((2, max_rows), dtype=torch.float32, device=device)
        self.ids = torch.empty(max_rows, dtype=torch.int32, device=device)     # the last draw, on the device
        self._ids_host = torch.empty((2, max_rows), dtype=torch.int32, pin_memory=True)
        self._events = [torch.cuda.Event(), torch.cuda.Event()]
        self._turn = 0

    def sample_async(self, logits, inv_temps, uniforms):
        """Enqueue the draw for ``logits`` float32 [R, V] (per row ``inv_temp``, <= 0: argmax, and a
        uniform number in [0, 1)).  The ids stay in ``self.ids`` for the next step and are copied
        to the host asynchronously; returns a handle for ``collect``."""
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
                h = self._host[k].numpy()
                h[0, :R] = inv_temps
                h[1, :R] = uniforms
                self._dev[0, :R].copy_(self._host[k, 0, :R], non_blocking=True)
                self._dev[1, :R].copy_(self._host[k, 1, :R], non_blocking=True)
                ops.sample(logits, self._dev[0, :R], self._dev[1, :R], ids)
            self._ids_host[k, :R].copy_(ids, non_blocking=True)
        self._events[k].record()
        return k, R

    def collect(self, handle) -> list:
        k, R = handle
        self._events[k].synchronize()
        return self._ids_host[k, :R].tolist()

    def sample(self, logits, inv_temps, uniforms) -> list:
        return self.collect(self.sample_async(logits, inv_temps, uniforms))
