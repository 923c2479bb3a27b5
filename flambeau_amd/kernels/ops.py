"""Typed wrappers of the plain kernels.

Each wrapper checks on the host that the tensors have the device, dtype, contiguity
and shape the kernel and its grid assume, and only then launches on torch's current
stream.  (The reference keeps the same split: typed, bounds-checked leaf functions
above raw launches, crates/model-ops/src/lib.rs:47-82.)
"""
from __future__ import annotations

from dataclasses import dataclass

import torch

from .library import KernelError, call

_DT = {torch.float32: 0, torch.bfloat16: 1}


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return _DT[dtype]
    except KeyError:
        raise KernelError(f"unsupported dtype {dtype}: the kernels take float32 and bfloat16") from None


_pinned_stream = None


def stream_handle() -> int:
    """The stream kernels are launched on: torch's current one, or the one pinned for a forward pass."""
    return _pinned_stream if _pinned_stream is not None else torch.cuda.current_stream().cuda_stream


class pinned_stream:
    """``with pinned_stream():`` every launch inside goes to the stream that is current on entry.
    Asking torch for its current stream at each of a step's two hundred launches costs more than
    the launches; nothing inside a forward pass changes the stream."""

    def __enter__(self):
        global _pinned_stream
        self.prev = _pinned_stream
        _pinned_stream = torch.cuda.current_stream().cuda_stream

    def __exit__(self, *exc):
        global _pinned_stream
        _pinned_stream = self.prev


def _check(t: torch.Tensor, name: str, dtype=None, shape=None):
    if not isinstance(t, torch.Tensor):
        raise KernelError(f"{name}: expected a tensor, got {type(t).__name__}")
    if not t.is_cuda:
        raise KernelError(f"{name}: tensor is on {t.device}, the kernels run on the GPU only")
    if not t.is_contiguous():
        raise KernelError(f"{name}: tensor is not contiguous")
    if dtype is not None and t.dtype != dtype:
        raise KernelError(f"{name}: dtype {t.dtype}, expected {dtype}")
    if shape is not None:
        have = t.shape
        ok = len(have) == len(shape)
        if ok:
            for s, e in zip(have, shape):
                if e is not None and e != s:
                    ok = False
                    break
        if not ok:
            raise KernelError(f"{name}: shape {tuple(have)}, expected {tuple(shape)}")
    return t.data_ptr()


@dataclass
class PagedLayerCache:
    """The key/value pool of one layer: ``pool[n_pages, 2, n_kv_heads, page_size, head_dim]``."""
    pool: torch.Tensor

    @property
    def n_pages(self): return self.pool.shape[0]
    @property
    def n_kv_heads(self): return self.pool.shape[2]
    @property
    def page_size(self): return self.pool.shape[3]
    @property
    def head_dim(self): return self.pool.shape[4]


def embed(table, tokens, out):
    V, H = table.shape
    n = tokens.shape[0]
    call("fl_embed", _check(table, "embed.table"), dtype_code(table.dtype),
         _check(tokens, "embed.tokens", torch.int32, (n,)),
         _check(out, "embed.out", torch.float32, (n, H)), n, H, V, stream_handle())
    return out


def gather_rows(src, rows, out):
    """``out[r] = src[rows[r]]`` for a float32 ``src`` (the embedding kernel over a table of rows)."""
    return embed(src, rows, out)


def rmsnorm(x, weight, out, eps, delta=None, store_sum=False, rows=None):
    """``out = rmsnorm(x (+ delta)) * weight``; ``store_sum`` writes x + delta back into x;
    ``rows`` (int32) picks the rows of x that are normed, one output row each."""
    n, H = x.shape
    px = _check(x, "rmsnorm.x", torch.float32, (n, H))
    pd = _check(delta, "rmsnorm.delta", torch.float32, (n, H)) if delta is not None else None
    pr = _check(rows, "rmsnorm.rows", torch.int32) if rows is not None else None
    n_out = rows.shape[0] if rows is not None else n
    if store_sum and delta is None:
        store_sum = False
    call("fl_rmsnorm", px, pd, px if store_sum else None, pr,
         _check(weight, "rmsnorm.weight", torch.float32, (H,)),
         _check(out, "rmsnorm.out", None, (n_out, H)), dtype_code(out.dtype), n_out, H, float(eps),
         stream_handle())
    return out


def add_inplace(x, delta):
    if x.shape != delta.shape:
        raise KernelError(f"add: shapes {tuple(x.shape)} and {tuple(delta.shape)} differ")
    call("fl_add_inplace", _check(x, "add.x", torch.float32), _check(delta, "add.delta", torch.float32),
         x.numel(), stream_handle())
    return x


def gemm_plain(x, w, out):
    """``out[m, n] = sum_k x[m, k] w[n, k]``."""
    M, K = x.shape
    N = w.shape[0]
    call("fl_gemm_plain", _check(x, "gemm.x", w.dtype, (M, K)), _check(w, "gemm.w", None, (N, K)),
         _check(out, "gemm.out", None, (M, N)), dtype_code(x.dtype), dtype_code(out.dtype), M, N, K,
         stream_handle())
    return out


def rope_table(positions, rotated_dims, theta, out):
    """``out[n, rotated_dims / 2, 2]`` = (cos, sin)(position * theta^(-2 i / rotated_dims)), float32."""
    n = positions.shape[0]
    call("fl_rope_table", _check(positions, "rope.positions", torch.int32, (n,)), n, int(rotated_dims), float(theta),
         _check(out, "rope.table", torch.float32, (n, rotated_dims // 2, 2)), stream_handle())
    return out


def rope_table_ladder(positions, rotated_dims, inv_freq, out, magnitude: float = 1.0):
    """``rope_table`` from frequencies of the caller's own: ``out[n, rotated_dims / 2, 2]`` = ``magnitude`` *
    (cos, sin)(position * inv_freq[i]); ``inv_freq``: float64 ``[rotated_dims / 2]`` on the device."""
    n = positions.shape[0]
    call("fl_rope_table_ladder", _check(positions, "rope.positions", torch.int32, (n,)), n, int(rotated_dims),
         _check(inv_freq, "rope.inv_freq", torch.float64, (rotated_dims // 2,)), float(magnitude),
         _check(out, "rope.table", torch.float32, (n, rotated_dims // 2, 2)), stream_handle())
    return out


def rope_kv_write(qkv, positions, tok_seq, block_table, q_out, cache: PagedLayerCache, n_heads,
                  rotated_dims, theta, write_cache=True, table=None, paired=False, parts: int = 1):
    """Rotate q and k, store q and the cache rows.  ``table``: the step's ``rope_table`` (else the
    angles are computed here); ``paired``: the projection's rows come in the order of
    ``rotary_paired_rows``.  With ``parts`` > 1 ``qkv`` is ``[parts, n, ld]``: partial sums of a
    product that split K, added here."""
    if parts > 1 or qkv.dim() == 3:
        if qkv.dim() != 3 or qkv.shape[0] != parts or not qkv.is_contiguous():
            raise KernelError(f"rope_kv_write: {parts} parts want a contiguous [{parts}, n, ld] tensor")
        part_stride = qkv.shape[1] * qkv.shape[2]
        n, ld = qkv.shape[1:]
    else:
        part_stride = 0
        n, ld = qkv.shape
    nkv, hd = cache.n_kv_heads, cache.head_dim
    if ld != (n_heads + 2 * nkv) * hd:
        raise KernelError(f"rope_kv_write: row of {ld} values, expected {(n_heads + 2 * nkv) * hd}")
    call("fl_rope_kv_write", _check(qkv, "rope.qkv"), dtype_code(qkv.dtype), ld,
         _check(positions, "rope.positions", torch.int32, (n,)),
         _check(tok_seq, "rope.tok_seq", torch.int32, (n,)),
         _check(block_table, "rope.block_table", torch.int32, (None, None)), block_table.shape[1],
         _check(q_out, "rope.q_out", cache.pool.dtype, (n, n_heads * hd)),
         _check(cache.pool, "rope.cache"), dtype_code(cache.pool.dtype), n, n_heads, nkv, hd,
         cache.page_size, cache.n_pages, int(rotated_dims), float(theta), int(bool(write_cache)),
         _check(table, "rope.table", torch.float32, (n, rotated_dims // 2, 2)) if table is not None and rotated_dims else None,
         int(bool(paired)), int(parts), int(part_stride), stream_handle())
    return q_out


def attn_plain(q, out, cache: PagedLayerCache, positions, tok_seq, block_table, n_heads, scale, window):
    n = q.shape[0]
    hd = cache.head_dim
    dt = cache.pool.dtype
    call("fl_attn_plain", _check(q, "attn.q", dt, (n, n_heads * hd)),
         _check(out, "attn.out", dt, (n, n_heads * hd)), _check(cache.pool, "attn.cache"),
         dtype_code(dt), _check(positions, "attn.positions", torch.int32, (n,)),
         _check(tok_seq, "attn.tok_seq", torch.int32, (n,)),
         _check(block_table, "attn.block_table", torch.int32, (None, None)), block_table.shape[1],
         n, n_heads, cache.n_kv_heads, hd, cache.page_size, cache.n_pages, float(scale), int(window),
         stream_handle())
    return out


def attention_max_head_dim() -> int:
    """The largest head size the attention kernels take (a host function: no GPU needed)."""
    from .library import load
    return load().fl_attn_max_head_dim()


def silu_mul(gu, out):
    n, two_i = gu.shape
    I = two_i // 2
    call("fl_silu_mul", _check(gu, "silu_mul.gu"), dtype_code(gu.dtype),
         _check(out, "silu_mul.out", None, (n, I)), dtype_code(out.dtype), n, I, stream_handle())
    return out


def feed_tokens(tokens, ids, src):
    """``tokens[i] = ids[src[i]]`` where ``src[i] >= 0``: ids drawn on the device in the step before."""
    n = tokens.shape[0]
    call("fl_feed_tokens", _check(tokens, "feed.tokens", torch.int32, (n,)), _check(ids, "feed.ids", torch.int32),
         _check(src, "feed.src", torch.int32, (n,)), n, stream_handle())
    return tokens


def argmax(logits, out):
    R, V = logits.shape
    call("fl_argmax", _check(logits, "argmax.logits", torch.float32), _check(out, "argmax.out", torch.int32, (R,)),
         R, V, stream_handle())
    return out


def _counts(counts, V):
    if counts.dtype != torch.int16 or counts.dim() != 2 or counts.shape[1] != V or not counts.is_contiguous() or not counts.is_cuda:
        raise KernelError(f"sample.counts: {counts.dtype} {tuple(counts.shape)}, want int16 [slots, {V}] on the device")
    return counts.data_ptr()


def sample_penalise(logits, counts, slot, repetition, presence, frequency):
    """Repetition, presence and frequency penalties in place on ``logits`` [R, V] for the rows with a
    history (``slot`` >= 0 as a float: row of ``counts``, int16 [slots, V], how often each token was
    generated)."""
    R, V = logits.shape
    f = lambda t, name: _check(t, "sample_penalise." + name, torch.float32, (R,))
    call("fl_sample_penalise", _check(logits, "sample_penalise.logits", torch.float32), R, V, _counts(counts, V),
         f(slot, "slot"), f(repetition, "repetition"), f(presence, "presence"), f(frequency, "frequency"), stream_handle())
    return logits


def sample_bias(logits, rows, tokens, values):
    """``logits[rows[j], tokens[j]] += values[j]`` (all float32 [n]; a pair occurs once)."""
    V, n = logits.shape[1], rows.shape[0]
    f = lambda t, name: _check(t, "sample_bias." + name, torch.float32, (n,))
    call("fl_sample_bias", _check(logits, "sample_bias.logits", torch.float32), V, n, f(rows, "rows"), f(tokens, "tokens"),
         f(values, "values"), stream_handle())
    return logits


def sample_count(counts, slot, ids):
    """The tokens ``ids`` drawn for the rows with a history join it: ``counts[slot[r], ids[r]] += 1``."""
    R, V = ids.shape[0], counts.shape[1]
    call("fl_sample_count", _counts(counts, V), V, R, _check(slot, "sample_count.slot", torch.float32, (R,)),
         _check(ids, "sample_count.ids", torch.int32, (R,)), stream_handle())


def sample_history(counts, slot: int, tokens):
    """Row ``slot`` of ``counts`` is zeroed and the ``tokens`` (int32 [n], may be empty) are counted."""
    V, n = counts.shape[1], tokens.shape[0]
    call("fl_sample_history", _counts(counts, V), V, int(slot),
         _check(tokens, "sample_history.tokens", torch.int32, (n,)) if n else None, n, stream_handle())


def sample_filtered(logits, inv_temp, uniform, top_k, top_p, min_p, out, stash=None):
    """The temperature draw through top-k, top-p and min-p for the rows that ask for them (``top_k``
    >= 1 as a float, 0 < ``top_p`` < 1, ``min_p`` > 0); other rows of ``out`` are not touched.
    ``stash`` (int32 or float32, at least R * V values): scratch that spares a vocabulary beyond 32,768
    the forming of its probabilities in every pass."""
    R, V = logits.shape
    if stash is not None and (stash.numel() < R * V or stash.element_size() != 4 or not stash.is_contiguous()):
        raise KernelError(f"sample_filtered.stash: {stash.numel()} values of {stash.element_size()} bytes, {R * V} of 4 wanted")
    f = lambda t, name: _check(t, "sample_filtered." + name, torch.float32, (R,))
    call("fl_sample_filtered", _check(logits, "sample_filtered.logits", torch.float32), f(inv_temp, "inv_temp"),
         f(uniform, "uniform"), f(top_k, "top_k"), f(top_p, "top_p"), f(min_p, "min_p"),
         _check(out, "sample_filtered.out", torch.int32, (R,)), R, V,
         stash.data_ptr() if stash is not None else None, stream_handle())
    return out


def sample(logits, inv_temp, uniform, out):
    R, V = logits.shape
    call("fl_sample", _check(logits, "sample.logits", torch.float32),
         _check(inv_temp, "sample.inv_temp", torch.float32, (R,)),
         _check(uniform, "sample.uniform", torch.float32, (R,)),
         _check(out, "sample.out", torch.int32, (R,)), R, V, stream_handle())
    return out
