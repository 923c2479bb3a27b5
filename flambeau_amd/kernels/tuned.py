"""Wrappers of the tuned bfloat16 kernels and the choice between them.

Every tuned kernel stands beside a plain one that computes the same thing; where a tuned
kernel does not take a shape (a K that is no multiple of 8, a head size beyond 256) the plain
kernel runs instead, so a size is never answered with a wrong result."""
from __future__ import annotations

import torch

from . import ops
from .library import P, I, F, call, register_signatures
from .ops import _check, dtype_code, stream_handle

register_signatures({
    "fl_gemm_skinny": [P, P, P, I, I, I, I, P],
})

SKINNY_MAX_ROWS = 64


def gemm_skinny(x, w, out):
    M, K = x.shape
    N = w.shape[0]
    call("fl_gemm_skinny", _check(x, "gemm.x", torch.bfloat16, (M, K)), _check(w, "gemm.w", torch.bfloat16, (N, K)),
         _check(out, "gemm.out", None, (M, N)), dtype_code(out.dtype), M, N, K, stream_handle())
    return out


def gemm(x, w, out):
    M, K = x.shape
    if x.dtype == torch.bfloat16 and K % 8 == 0:
        if M <= SKINNY_MAX_ROWS:
            return gemm_skinny(x, w, out)
    return ops.gemm_plain(x, w, out)


def attention_metadata(batch) -> dict:
    return {}


def attention(q, out, cache, step, table, n_heads, scale, window):
    return ops.attn_plain(q, out, cache, step.positions, step.tok_seq, table, n_heads, scale, window)
