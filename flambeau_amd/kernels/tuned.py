"""Dispatch to the tuned bfloat16 kernels (plain kernels where no tuned one exists yet)."""
from __future__ import annotations

from . import ops


def gemm(x, w, out):
    return ops.gemm_plain(x, w, out)


def attention_metadata(batch) -> dict:
    return {}


def attention(q, out, cache, step, table, n_heads, scale, window):
    return ops.attn_plain(q, out, cache, step.positions, step.tok_seq, table, n_heads, scale, window)
