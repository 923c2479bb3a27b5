"""Split-half rotary position encoding.

pair i in [0, rot/2): f_i = theta^(-2i/rot), phi = pos * f_i,
(x[i], x[i+rot/2]) <- (x[i]cos(phi) - x[i+rot/2]sin(phi), x[i]sin(phi) + x[i+rot/2]cos(phi)),
in 32-bit (crates/kernels-hip/src/kernels/rope_neox_partial_f16.cu:37-52).  The rotation
itself runs inside the mixer's rotate-and-store kernel; this part only carries its
constants."""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import POSITION_ENCODINGS, PositionEncoding


@POSITION_ENCODINGS.register("rope_neox")
class RotaryNeoX(PositionEncoding):
    replayable = True

    def __init__(self, head_dim: int, theta: float, rotated_dims: int | None = None):
        self.head_dim = head_dim
        self.theta = float(theta)
        self.rotated_dims = head_dim if rotated_dims is None else rotated_dims
        if self.rotated_dims % 2 or not 0 < self.rotated_dims <= head_dim:
            raise ValueError(f"rotated dims {self.rotated_dims} must be even and within the head size {head_dim}")

    def rotary_parameters(self):
        return self.rotated_dims, self.theta

    def inverse_frequencies(self):
        """``None``: the ladder ``theta^(-2 i / rotated_dims)``.  A subclass with another ladder (scaled,
        interpolated, cut) returns its ``rotated_dims / 2`` frequencies (floats, made in double) and
        may set ``magnitude``, a factor on every cosine and sine; everything else stays: the table is
        made from them, and the kernels that rotate read the table."""
        return None

    magnitude = 1.0

    def bind(self, weights, rt):
        self.rt = rt
        freqs = self.inverse_frequencies()
        self._ladder = None
        if freqs is not None:
            if len(freqs) != self.rotated_dims // 2:
                raise ValueError(f"{len(freqs)} frequencies for {self.rotated_dims} rotated dims")
            self._ladder = torch.tensor([float(f) for f in freqs], dtype=torch.float64, device=rt.device)
            self._ladder_key = tuple(float(f) for f in freqs)

    def rotary_table(self, rt, step):
        """The angles depend on the positions only: their cosines and sines are made once per
        forward pass and shared by all layers with the same constants."""
        ladder = getattr(self, "_ladder", None)
        key = ("rope_neox", self.rotated_dims, self.theta if ladder is None else self._ladder_key, self.magnitude)
        table = step.scratch.get(key)
        if table is None:
            half = self.rotated_dims // 2
            name = f"rope_table_{self.rotated_dims}_{self.theta}" if ladder is None else f"rope_table_{hash(key)}"
            table = rt.buffer(name, step.n_tokens, 2 * half, torch.float32)
            table = table.view(step.n_tokens, half, 2)
            if ladder is None:
                ops.rope_table(step.positions, self.rotated_dims, self.theta, table)
            else:
                ops.rope_table_ladder(step.positions, self.rotated_dims, ladder, table, self.magnitude)
            step.scratch[key] = table
        return table


@POSITION_ENCODINGS.register("none")
class NoPositionEncoding(PositionEncoding):
    replayable = True

    def __init__(self, **_):
        pass

    def rotary_parameters(self):
        return 0, 1.0
