"""Split-half rotary position encoding.

pair i in [0, rot/2): f_i = theta^(-2i/rot), phi = pos * f_i,
(x[i], x[i+rot/2]) <- (x[i]cos(phi) - x[i+rot/2]sin(phi), x[i]sin(phi) + x[i+rot/2]cos(phi)),
in 32-bit (crates/kernels-hip/src/kernels/rope_neox_partial_f16.cu:37-52).  The rotation
itself runs inside the mixer's rotate-and-store kernel; this part only carries its
constants."""
from __future__ import annotations

from .base import POSITION_ENCODINGS, PositionEncoding


@POSITION_ENCODINGS.register("rope_neox")
class RotaryNeoX(PositionEncoding):
    def __init__(self, head_dim: int, theta: float, rotated_dims: int | None = None):
        self.head_dim = head_dim
        self.theta = float(theta)
        self.rotated_dims = head_dim if rotated_dims is None else rotated_dims
        if self.rotated_dims % 2 or not 0 < self.rotated_dims <= head_dim:
            raise ValueError(f"rotated dims {self.rotated_dims} must be even and within the head size {head_dim}")

    def rotary_parameters(self):
        return self.rotated_dims, self.theta


@POSITION_ENCODINGS.register("none")
class NoPositionEncoding(PositionEncoding):
    def __init__(self, **_):
        pass

    def rotary_parameters(self):
        return 0, 1.0
