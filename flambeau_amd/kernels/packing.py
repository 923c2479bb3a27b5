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


def interleave_gate_up(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """Gate and up rows interleaved in fours, ``[g0-3 | u0-3 | g4-7 | u4-7]`` per eight features
    (I padded to a multiple of 8 with zero rows): one matrix-core tile of 16 rows then holds
    gate and up of the same eight features, and a kernel can apply ``silu(gate) * up`` before
    it stores."""
    I, K = gate.shape
    Ip = -(-I // 8) * 8
    if Ip != I:
        pad = torch.zeros((Ip - I, K), dtype=gate.dtype, device=gate.device)
        gate, up = torch.cat([gate, pad]), torch.cat([up, pad])
    g, u = gate.view(Ip // 8, 2, 4, K), up.view(Ip // 8, 2, 4, K)
    return torch.stack([g[:, 0], u[:, 0], g[:, 1], u[:, 1]], dim=1).reshape(2 * Ip, K).contiguous()


@dataclass
class Weight:
    """A matrix ``[rows, cols]`` (out features, in features) as the kernels take it: row-major,
    packed, or both."""
    rows: int
    cols: int
    rowmajor: torch.Tensor | None = None
    packed: torch.Tensor | None = None
    packed_rows: int = 0          # rows the packed form was built from (with interleaving and padding)
    swiglu_cols: int = 0          # > 0: the packed form holds interleaved gate/up rows of this many features

    @property
    def shape(self):
        return (self.rows, self.cols)

    @property
    def dtype(self):
        return (self.packed if self.packed is not None else self.rowmajor).dtype


def rotary_paired_rows(n_heads: int, n_kv_heads: int, head_dim: int, rotated_dims: int):
    """Order of the rows of a joined q/k/v projection in which a split-half rotation can be applied
    by the product's own kernel: within every q and k head the rotated dims come as 8 dims, their 8
    partners (dim + rotated_dims / 2), the next 8 dims, ...; a group of 16 output features then
    holds whole pairs, four lanes apart in the accumulators.  Dims beyond the rotated ones and the
    v heads keep their places.  ``perm[new row] = old row``; ``None`` if the sizes are not in
    steps of 16."""
    if rotated_dims <= 0 or rotated_dims % 16 or head_dim % 16:
        return None
    half = rotated_dims // 2
    head = []
    for b in range(half // 8):
        head += list(range(8 * b, 8 * b + 8)) + list(range(half + 8 * b, half + 8 * b + 8))
    head += list(range(rotated_dims, head_dim))
    perm = []
    for h in range(n_heads + n_kv_heads):
        perm += [h * head_dim + d for d in head]
    perm += list(range((n_heads + n_kv_heads) * head_dim, (n_heads + 2 * n_kv_heads) * head_dim))
    return torch.tensor(perm, dtype=torch.long)
