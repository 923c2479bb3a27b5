"""Arrangements of parts in a layer, and the residual stream they advance.

Pre-norm decoder layer: x += Mixer(Norm1(x)); x += FeedForward(Norm2(x))
(crates/forward/README.md:28-40; crates/models/qwen35-v2/src/model.rs:19-50).  The residual
stream is kept in 32-bit.  A delta is not added at once: it stays pending until the next norm,
which adds it, stores the sum and norms it in one kernel
(crates/kernels-hip/src/kernels/rmsnorm_f16_add_residual.cu)."""
from __future__ import annotations

from ..kernels import ops
from .base import BLOCKS, FEED_FORWARDS, MIXERS, NORMS, Block, PartSpec, Product


class ResidualStream:
    def __init__(self, resid, rt):
        self.resid = resid          # float32 [n, hidden]
        self.rt = rt
        self.pending = None         # float32 [n, hidden] not yet added, or a Product not yet computed

    def push(self, delta):
        """``delta``: what a part returned, a tensor or a ``Product``."""
        self.flush()
        self.pending = delta

    def _pending_tensor(self):
        if isinstance(self.pending, Product):
            self.pending = self.pending.compute(self.rt)
        return self.pending

    def flush(self):
        if self._pending_tensor() is not None:
            ops.add_inplace(self.resid, self.pending)
            self.pending = None
        return self.resid

    def normed(self, norm, rows=None, name="normed", lazy=False):
        """The normed stream in the compute dtype, the pending delta added on the way.  With
        ``lazy`` the caller takes what ``Norm.after_product`` returns as well as a tensor."""
        n, H = self.resid.shape
        if lazy and rows is None and isinstance(self.pending, Product):
            fused = norm.after_product(self.rt, self.resid, self.pending)
            if fused is not None:
                self.pending = None
                return fused
        self._pending_tensor()
        if rows is not None:
            out = self.rt.buffer(name + "_rows", rows.shape[0], H)
            norm.forward(self.resid, out, delta=self.pending, rows=rows)
            return out
        out = self.rt.buffer(name, n, H)
        norm.forward(self.resid, out, delta=self.pending, store_sum=True)
        self.pending = None
        return out


@BLOCKS.register("prenorm")
class PreNormBlock(Block):
    replayable = True

    def __init__(self, mixer: PartSpec, feed_forward: PartSpec, norm: PartSpec):
        self.mixer_norm = NORMS.create(norm)
        self.mixer = MIXERS.create(mixer)
        self.ffn_norm = NORMS.create(norm)
        self.ffn = FEED_FORWARDS.create(feed_forward)
        self._parts = {"mixer_norm": self.mixer_norm, "mixer": self.mixer,
                       "ffn_norm": self.ffn_norm, "ffn": self.ffn}

    def cache_spec(self):
        return self.mixer.cache_spec()

    def mixers(self):
        return [self.mixer]

    def subparts(self):
        return list(self._parts.values())

    def tensors(self):
        return {f"{p}.{name}": spec for p, part in self._parts.items() for name, spec in part.tensors().items()}

    def bind(self, weights, rt):
        self.rt = rt
        for p, part in self._parts.items():
            part.bind({k[len(p) + 1:]: v for k, v in weights.items() if k.startswith(p + ".")}, rt)

    def forward(self, stream, step, cache):
        stream.push(self.mixer.forward(stream.normed(self.mixer_norm, lazy=self.mixer.lazy_input), step, cache))
        stream.push(self.ffn.forward(stream.normed(self.ffn_norm, lazy=self.ffn.lazy_input), step))
