"""Weight matrices in the layout the matrix cores read them in.

``pack_weight`` turns a row-major ``[N, K]`` bfloat16 matrix into tiles of 16 rows x 32 k:
each tile is the A (or B) operand of one ``v_mfma_f32_16x16x32_bf16`` laid out in lane order
(lane ``16 g + i`` holds row ``i``, k ``8 g .. 8 g + 7``), i.e. 1 KB of contiguous memory; the
tiles of a group of 16 rows follow each other along k, the row groups follow each other.
N is padded to a multiple of 16 and K to a multiple of 32 with zeros.  The permutation is
done once when the weights are loaded.
"""
from __future__ import annotations

from dataclasses import dataclass

import torch


def pack_weight(w: torch.Tensor) -> torch.Tensor:
    N, K = w.shape
    Np, Kp = -(-N // 16) * 16, -(-K // 32) * 32
    if (Np, Kp) != (N, K):
        wp = torch.zeros((Np, Kp), dtype=w.dtype, device=w.device)
        wp[:N, :K] = w
        w = wp
    t = w.view(Np // 16, 16, Kp // 32, 4, 8).permute(0, 2, 3, 1, 4)      # [row group, step, g, i, e]
    return t.contiguous().view(-1)


def unpack_weight(packed: torch.Tensor, N: int, K: int) -> torch.Tensor:
    Np, Kp = -(-N // 16) * 16, -(-K // 32) * 32
    t = packed.view(Np // 16, Kp // 32, 4, 16, 8).permute(0, 3, 1, 2, 4).reshape(Np, Kp)
    return t[:N, :K].contiguous()


@dataclass
class Weight:
    """A matrix ``[rows, cols]`` (out features, in features) as the kernels take it: row-major,
    packed, or both."""
    rows: int
    cols: int
    rowmajor: torch.Tensor | None = None
    packed: torch.Tensor | None = None

    @property
    def shape(self):
        return (self.rows, self.cols)

    @property
    def dtype(self):
        return (self.packed if self.packed is not None else self.rowmajor).dtype
